"""The tiled weight copies that the matrix-core GEMVs read (the second resident format of Q4_K, Q4_0, Q8_0 and fp16 matrices): read
back from the GPU and compared byte for byte with tiles rebuilt here from the GGUF blocks by the layouts' definitions, ragged row
counts included, so that the copy is held to the same bit-exactness as the row-major one that esp_matrix_dequantize reads."""
import numpy as np
import pytest

from oracle import oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import espresso_amd.ops as o
    o.init()
    return o


def weights(rows, cols, seed):
    return np.random.default_rng(seed).normal(0, 0.05, (rows, cols)).astype(np.float32)


def padded_rows(a, rows):
    """Rows past the matrix are zero blocks."""
    full = -(-rows // 16) * 16
    out = np.zeros((full,) + a.shape[1:], a.dtype)
    out[:rows] = a
    return out


@pytest.mark.parametrize("rows,cols", [(16, 4096), (37, 1024), (100, 14336), (48, 2048)])
def test_q4k_tiles(ops, rows, cols):
    """Tile (row block, super-block) = 2304 bytes: the sixteen rows' 16-byte headers, then for lane group g and row n the first 16 bytes of
    the 32-byte chunk g at 256 + 16 (16 g + n) and its second 16 bytes at 1280 + 16 (16 g + n)."""
    blocks = orc.quantize(orc.FMT_Q4_K, weights(rows, cols, rows))
    mat = ops.Matrix(orc.FMT_Q4_K, blocks, rows, cols)
    got = mat.read_tiled()
    nsb = cols // 256
    sb = padded_rows(np.asarray(blocks, np.uint8).reshape(rows, nsb, 144), rows)            # [row][super-block][144]
    rb = sb.reshape(-1, 16, nsb, 144).transpose(0, 2, 1, 3)                                   # [row block][super-block][n][144]
    want = np.zeros(rb.shape[:2] + (2304,), np.uint8)
    want[..., :256] = rb[..., :16].reshape(rb.shape[:2] + (256,))
    chunks = rb[..., 16:].reshape(rb.shape[:3] + (4, 2, 16))                                  # [..][n][g][half][16]
    for half in range(2):
        piece = chunks[..., half, :].transpose(0, 1, 3, 2, 4)                                 # [..][g][n][16]
        want[..., 256 + 1024 * half:256 + 1024 * (half + 1)] = piece.reshape(rb.shape[:2] + (1024,))
    assert got.size == want.size == mat.resident_bytes - mat.bytes
    assert np.array_equal(got, want.reshape(-1))
    mat.close()


@pytest.mark.parametrize("rows,cols", [(16, 4096), (21, 4096), (40, 14336)])
def test_q40_tiles(ops, rows, cols):
    """Tile (row block, 512 columns) = 4608 bytes: [j][lane = 16 g + n] the sixteen nibble bytes of block 16 t + 4 j + g of row n, then
    [lane][j] their fp16 scales."""
    blocks = np.asarray(orc.quantize(orc.FMT_Q4_0, weights(rows, cols, rows)), np.uint8).reshape(rows, cols // 32, 18)
    mat = ops.Matrix(orc.FMT_Q4_0, blocks.reshape(-1), rows, cols)
    got = mat.read_tiled()
    tpr = cols // 512
    b = padded_rows(blocks, rows).reshape(-1, 16, tpr, 4, 4, 18)                              # [row block][n][t][j][g][18]
    want = np.zeros((b.shape[0], tpr, 4608), np.uint8)
    nib = b[..., 2:].transpose(0, 2, 3, 4, 1, 5)                                              # [rb][t][j][g][n][16]
    want[..., :4096] = nib.reshape(b.shape[0], tpr, 4096)
    sc = b[..., :2].transpose(0, 2, 4, 1, 3, 5)                                               # [rb][t][g][n][j][2]
    want[..., 4096:] = sc.reshape(b.shape[0], tpr, 512)
    assert got.size == want.size
    assert np.array_equal(got, want.reshape(-1))
    mat.close()


@pytest.mark.parametrize("rows,cols", [(16, 768), (50, 2048), (33, 4096)])
def test_q80_tiles(ops, rows, cols):
    """Tile (row block, 256 columns) = 4352 bytes: [j][half][lane = 16 g + n] sixteen quants (first or last half) of block 8 t + 4 j + g of
    row n, then per lane the fp16 scales of its blocks j = 0 and j = 1."""
    blocks = np.asarray(orc.quantize(orc.FMT_Q8_0, weights(rows, cols, rows)), np.uint8).reshape(rows, cols // 32, 34)
    mat = ops.Matrix(orc.FMT_Q8_0, blocks.reshape(-1), rows, cols)
    got = mat.read_tiled()
    tpr = cols // 256
    b = padded_rows(blocks, rows).reshape(-1, 16, tpr, 2, 4, 34)                              # [rb][n][t][j][g][34]
    want = np.zeros((b.shape[0], tpr, 4352), np.uint8)
    q = b[..., 2:].reshape(b.shape[:5] + (2, 16)).transpose(0, 2, 3, 5, 4, 1, 6)              # [rb][t][j][half][g][n][16]
    want[..., :4096] = q.reshape(b.shape[0], tpr, 4096)
    sc = b[..., :2].transpose(0, 2, 4, 1, 3, 5)                                               # [rb][t][g][n][j][2]
    want[..., 4096:] = sc.reshape(b.shape[0], tpr, 256)
    assert got.size == want.size
    assert np.array_equal(got, want.reshape(-1))
    mat.close()


@pytest.mark.parametrize("rows,cols", [(16, 768), (45, 2048)])
def test_f16_tiles(ops, rows, cols):
    """Tile (row block, 256 columns) = 8192 bytes: [j][m][lane = 16 g + n] eight weights of row n, columns 32 (4 j + g) + 8 m .. + 7 of the
    tile, the middle two of every four exchanged."""
    w = weights(rows, cols, rows).astype(np.float16)
    mat = ops.Matrix(orc.FMT_F16, w.view(np.uint8).reshape(-1), rows, cols)
    got = mat.read_tiled()
    tpr = cols // 256
    a = padded_rows(w.view(np.uint16), rows).reshape(-1, 16, tpr, 2, 4, 4, 2, 4)              # [rb][n][t][j][g][m][four][4]
    a = a[..., [0, 2, 1, 3]]
    want = a.transpose(0, 2, 3, 5, 4, 1, 6, 7).reshape(-1)                                    # [rb][t][j][m][g][n][8]
    assert got.size == want.size * 2
    assert np.array_equal(got.view(np.uint16), want)
    mat.close()


def test_matrices_without_a_tiled_copy_report_none(ops):
    blocks = orc.quantize(orc.FMT_Q4_K, weights(16, 512, 1))
    mat = ops.Matrix(orc.FMT_Q4_K, blocks, 16, 512)
    assert mat.read_tiled().size == 0 and mat.resident_bytes == mat.bytes
    mat.close()
