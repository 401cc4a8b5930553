"""The reference runner's `<gguf> <tokenizer-dir> <prompt> [max]` form (Sources/EspressoGGUFRunner/main.swift:43-57 over
RunGGUF.main, Sources/EspressoGGUF/RunGGUF.swift:68-113): generated text on stdout, what the reference reports about the
run on stderr.

    python -m espresso_amd.run_gguf model.gguf tokenizer-dir "Hello" 32
"""
from __future__ import annotations

import os
import sys


def main(argv: list[str]) -> int:
    if len(argv) < 3:
        sys.stderr.write("Usage: python -m espresso_amd.run_gguf <gguf-path> <tokenizer-dir> <prompt> [max-tokens]\n")
        return 1
    try:
        max_tokens = int(argv[3]) if len(argv) > 3 else 32
    except ValueError:
        max_tokens = 32
    from . import engine as eng
    from . import ops
    try:
        ops.init()
        r = eng.run_gguf(argv[0], argv[1], argv[2], max_tokens, dict(os.environ))
    except Exception as e:   # the reference prints the error and exits with 1
        sys.stderr.write(f"Error: {e}\n")
        return 1
    c = r["config"]
    sys.stderr.write(f"Prepared: {c.name}, {c.n_layer} layers, d={c.d_model}, vocab={c.vocab}, {r['tensor_count']} tensors in {r['prepare_ms']:.0f}ms\n")
    sys.stderr.write("Architecture: llama\n")
    sys.stderr.write(f"Weight dir: {r['weight_dir']}\n")
    sys.stderr.write(f"Engine built in {r['build_ms']:.0f}ms\n")
    sys.stderr.write(f'Generating from prompt: "{argv[2]}"\n')
    print(r["text"])
    sys.stderr.write("\n--- Stats ---\n")
    sys.stderr.write(f"Tokens generated: {len(r['tokens'])}\n")
    sys.stderr.write(f"Tokens/sec: {r['tokens_per_second']:.2f}\n")
    sys.stderr.write(f"Compile time: {r['compile_time_ms']:.0f}ms\n")
    sys.stderr.write(f"First token latency: {r['first_token_latency_ms']:.2f}ms\n")
    if r["kept_weight_dir"]:
        sys.stderr.write(f"Keeping weight dir: {r['weight_dir']}\n")
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
