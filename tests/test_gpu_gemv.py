"""Decode GEMV through the C ABI (oilhip_gemv_f32) against the CPU oracle.

Tolerance (north star): relative L2 error <= 1e-5 against the double-precision
dot of the bit-exact decoded weights.  The reference's own FP32 summation order
is measured against the same yardstick for comparison."""
import os

import numpy as np
import pytest
import torch

import innova_amd as ia
import oracle as O
from gpu_util import gaussian_weights, rel_l2, to_orc_blocks

pytestmark = pytest.mark.gpu
TOL = 1e-5
GV = np.load(os.path.join(os.path.dirname(__file__), "golden", "block_gemv.npz"))


def run_case(fmts, rows, cols, M, seed, general=False, outlier_every=13):
    w = gaussian_weights(rows * cols, seed, outlier_every=outlier_every)
    payload, blocks = ia.block_codec.quantize_tensor(w, fmts)
    X = np.random.default_rng(seed + 1).standard_normal((M, cols)).astype(np.float32)
    with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
        got = dw.gemv(torch.from_numpy(X).cuda(), general=general).cpu().numpy()
    want = O.block_gemm(payload, to_orc_blocks(blocks), rows, cols, X, wide=True)
    assert got.shape == (M, rows)
    return rel_l2(got, want), payload, blocks, X, want


@pytest.mark.parametrize("name", list(O.FORMATS))
def test_golden_gemv_every_format(name):
    """Reference payloads + double-precision outputs of the reference-decoded weights."""
    rows, cols, B = (int(v) for v in GV["shape"])
    il, cl = GV[f"{name}/idx_len"], GV[f"{name}/cb_len"]
    payload = np.concatenate([GV[f"{name}/idx"], GV[f"{name}/cb"], np.zeros(16, np.uint8)])
    blocks = np.zeros(il.size, dtype=ia._lib.BLOCK_DTYPE)
    blocks["idx_off"] = np.concatenate([[0], np.cumsum(il)[:-1]])
    blocks["idx_bytes"] = il
    blocks["cb_off"] = GV[f"{name}/idx"].size + np.concatenate([[0], np.cumsum(cl)[:-1]])
    blocks["cb_bytes"] = cl
    blocks["nw"], blocks["fmt"] = 256, O.FORMATS[name]
    X = GV["x_bits"].view(np.float32).reshape(B, cols)
    want = GV[f"{name}/y_bits"].view(np.float32).reshape(B, rows)
    with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
        got = dw.gemv(torch.from_numpy(X.copy()).cuda()).cpu().numpy()
        gen = dw.gemv(torch.from_numpy(X.copy()).cuda(), general=True).cpu().numpy()
    assert rel_l2(got, want) <= TOL, name
    assert rel_l2(gen, want) <= TOL, name


@pytest.mark.parametrize("fmt", list(ia.Format))
@pytest.mark.parametrize("M", [1, 3])
def test_uniform_format_gemv(fmt, M):
    err, *_ = run_case(fmt, rows=70, cols=1280, M=M, seed=20 + int(fmt))
    assert err <= TOL


def test_mixed_format_rows():
    rng = np.random.default_rng(3)
    rows, cols = 48, 2048
    fmts = rng.integers(0, 15, rows * cols // 256).astype(np.uint8)
    err, *_ = run_case(fmts, rows, cols, M=2, seed=31)
    assert err <= TOL


# rows that mix formats run on the tile- and format-ordered layout: the planner's half-and-half SPARK_Q0 / OIL1 plan,
# the four-format stress plan, the grouped mixes and all fifteen formats at once; row counts that are not a multiple
# of the tile, single-block rows, one to nine activation rows, streams of several windows, and rows too wide for the
# window-stream kernel's LDS (they fall back to the descriptor-driven kernel)
@pytest.mark.parametrize("fmt_ids", [(0, 1), (0, 1, 2, 3), (7, 9, 10, 11), (6, 11, 9, 7), tuple(range(15))])
@pytest.mark.parametrize("rows,cols,M", [(4, 256, 1), (7, 512, 2), (33, 4096, 1), (130, 2816, 3), (61, 1024, 5), (1, 1536, 4),
                                          (20, 768, 9), (3000, 512, 1), (9, 25600, 2)])
def test_mixed_format_tiles(fmt_ids, rows, cols, M):
    rng = np.random.default_rng(rows * 7 + cols + M + len(fmt_ids))
    fmts = rng.choice(np.array(fmt_ids, dtype=np.uint8), size=rows * cols // 256)
    if fmts.min() == fmts.max():
        fmts[0] = fmt_ids[0] if fmts[0] != fmt_ids[0] else fmt_ids[1]
    err, payload, blocks, X, want = run_case(fmts, rows, cols, M=M, seed=57 + rows)
    assert err <= TOL
    with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:      # the reordered payload decodes as before
        got = dw.dequant().cpu().numpy()
    ref = O.dequant_blocks(payload, to_orc_blocks(blocks))
    assert np.array_equal(got.view(np.uint32).ravel(), ref.view(np.uint32).ravel())


def test_mixed_format_skewed_tiles():
    """Tiles in which a format is absent, or holds a single block, or fills every block."""
    rows, cols = 24, 2048
    fmts = np.zeros(rows * cols // 256, dtype=np.uint8)          # OIL1 everywhere ...
    fmts[8 * 8: 12 * 8] = 1                                      # ... rows 8-11 all SPARK_Q0 (one whole tile)
    fmts[5] = 3                                                  # a single OIL4 block in tile 0
    fmts[-1] = 11                                                # a single OIL8_GRP block in the last row
    err, *_ = run_case(fmts, rows, cols, M=1, seed=77)
    assert err <= TOL


# the fast OIL4 kernel: every slab width (cols/256 = 16 -> 8 blocks per slab, 43 -> 4,
# 6 -> 2, 3 -> 1, 56 -> 8), ragged row counts, chunked rows, M up to 16
@pytest.mark.parametrize("rows,cols", [(64, 4096), (1000, 4096), (37, 11008), (300, 11008),
                                        (129, 1536), (50, 768), (77, 14336), (1, 256), (5, 512),
                                        (3000, 2048)])
@pytest.mark.parametrize("M", [1, 2, 4, 16])
def test_oil4_fast_kernel_shapes(rows, cols, M):
    if M > 2 and rows * cols > 2_000_000:
        pytest.skip("large-M cases are covered at the smaller shapes")
    err, payload, blocks, X, want = run_case(ia.Format.OIL4, rows, cols, M, seed=rows + cols + M)
    assert err <= TOL
    ref32 = O.block_gemm(payload, to_orc_blocks(blocks), rows, cols, X, wide=False)
    # the reference's own FP32 order sits at a comparable distance from the yardstick
    assert rel_l2(ref32, want) <= TOL


# the multi-token kernel: passes of 32 tokens (two token tiles), of 16 and of 8 or fewer (alone and as the last pass of a batch), several
# row tiles per workgroup (rows > 48 * 256), several K-slabs, an odd number of blocks per row
@pytest.mark.parametrize("rows,cols", [(130, 4096), (61, 11008), (13000, 512), (47, 14336), (3, 256)])
@pytest.mark.parametrize("M", [3, 5, 8, 9, 13, 17, 32, 33, 40, 70])
def test_oil4_multi_token_counts(rows, cols, M):
    err, *_ = run_case(ia.Format.OIL4, rows, cols, M, seed=7 * rows + cols + M)
    assert err <= TOL


# rows wider than 16 blocks are cut along K between workgroups whose sums meet in a workspace and are added in a fixed
# order (the output buffer holds NaNs before the call), several row tiles per workgroup, parts of unequal length, both
# pass widths
@pytest.mark.parametrize("rows,cols,M", [(9000, 8192, 5), (9000, 8192, 17), (5000, 11008, 16), (700, 8448, 24)])
def test_oil4_multi_token_rows_cut_along_k(rows, cols, M):
    w = gaussian_weights(rows * cols, rows + M)
    payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL4)
    X = np.random.default_rng(rows + M + 1).standard_normal((M, cols)).astype(np.float32)
    want = O.block_gemm(payload, to_orc_blocks(blocks), rows, cols, X, wide=True)
    with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
        out = torch.full((M, rows), float("nan"), device="cuda")
        runs = []
        for _ in range(3):                                   # later calls find the earlier calls' sums in y and in the workspace
            got = dw.gemv(torch.from_numpy(X).cuda(), out=out).cpu().numpy()
            assert rel_l2(got, want) <= TOL
            runs.append(got.copy())
        # the parts are added in a fixed order: the same bits from every launch
        assert np.array_equal(runs[0].view(np.uint32), runs[1].view(np.uint32))
        assert np.array_equal(runs[0].view(np.uint32), runs[2].view(np.uint32))


# the OIL8 kernel: one and several slabs per row, rows not a multiple of the wave count, several chunks per
# wavefront (tall tensors), every activation-row grouping, a partial last column set
@pytest.mark.parametrize("rows,cols", [(64, 4096), (1000, 4096), (37, 11008), (300, 1024), (5000, 256), (3, 256),
                                       (40000, 512), (4096, 4096), (130, 14336), (77, 2304)])
@pytest.mark.parametrize("M", [1, 2, 3, 4])
def test_oil8_fast_kernel_shapes(rows, cols, M):
    if rows * cols > 16e6 and M > 1:
        pytest.skip("the large shapes run once")
    err, payload, blocks, X, want = run_case(ia.Format.OIL8, rows, cols, M, seed=3 * rows + cols + M)
    assert err <= TOL


@pytest.mark.parametrize("rows,cols,M", [(1000, 4096, 6), (300, 1024, 9), (37, 11008, 5), (4096, 4096, 16)])
def test_oil8_more_than_four_activation_rows(rows, cols, M):
    """Batches beyond four rows run as consecutive launches of four rows or fewer."""
    err, *_ = run_case(ia.Format.OIL8, rows, cols, M, seed=5 * rows + cols + M)
    assert err <= TOL


def test_oil8_special_blocks():
    """Zero blocks, underflowing scales, huge outliers, zero activations, activations with a large common offset
    (the kernel forms sum(q x) - 127.5 sum(x), which must not lose the small difference)."""
    rows, cols = 96, 4096
    w = gaussian_weights(rows * cols, 177)
    w[0:256] = 0.0
    w[256 * 20: 256 * 21] *= np.float32(1e-7)
    w[256 * 40: 256 * 41] *= np.float32(1e4)
    payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL8)
    rng = np.random.default_rng(178)
    for offset in (0.0, 30.0):
        X = (rng.standard_normal((2, cols)) + offset).astype(np.float32)
        X[0, ::5] = 0.0
        with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
            got = dw.gemv(torch.from_numpy(X).cuda()).cpu().numpy()
            gen = dw.gemv(torch.from_numpy(X).cuda(), general=True).cpu().numpy()
        want = O.block_gemm(payload, to_orc_blocks(blocks), rows, cols, X, wide=True)
        assert rel_l2(gen, want) <= TOL
        assert rel_l2(got, want) <= TOL


def test_oil4_special_blocks():
    """Zero blocks (-0.0 levels), underflowing scales, huge outliers, zero activations."""
    rows, cols = 96, 4096
    w = gaussian_weights(rows * cols, 77)
    w[0:256] = 0.0
    w[256 * 20: 256 * 21] *= np.float32(1e-7)
    w[256 * 40: 256 * 41] *= np.float32(1e4)
    payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL4)
    X = np.random.default_rng(78).standard_normal((1, cols)).astype(np.float32)
    X[0, ::5] = 0.0
    with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
        got = dw.gemv(torch.from_numpy(X).cuda()).cpu().numpy()
        gen = dw.gemv(torch.from_numpy(X).cuda(), general=True).cpu().numpy()
    want = O.block_gemm(payload, to_orc_blocks(blocks), rows, cols, X, wide=True)
    assert rel_l2(got, want) <= TOL and rel_l2(gen, want) <= TOL


@pytest.mark.parametrize("rows,cols", [(11008, 4096), (4096, 11008)])
@pytest.mark.parametrize("M", [1, 4, 16])
def test_oil4_llama_mlp_shapes_full_size(rows, cols, M):
    """Config sizes.  The oracle runs on a row sample; all rows are covered by
    linearity: y(x1 + x2) = y(x1) + y(x2) and y(2x) = 2 y(x) within tolerance."""
    w = gaussian_weights(rows * cols, seed=rows)
    payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL4)
    assert payload.size == 22544384
    rng = np.random.default_rng(cols + M)
    X = rng.standard_normal((M, cols)).astype(np.float32)
    with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
        xd = torch.from_numpy(X).cuda()
        y = dw.gemv(xd).cpu().numpy()
        y2 = dw.gemv(xd * 2.0).cpu().numpy()
        perm = torch.from_numpy(rng.permutation(M)).cuda()
        ysum = dw.gemv(xd + xd[perm]).cpu().numpy()
    assert rel_l2(y2, 2.0 * y) <= 1e-6
    assert rel_l2(ysum, y + y[perm.cpu().numpy()]) <= TOL
    # oracle on every 64th row and the last rows
    sel = np.unique(np.concatenate([np.arange(0, rows, 64), np.arange(rows - 8, rows)]))
    bpr = cols // 256
    ob = to_orc_blocks(blocks).reshape(rows, bpr)[sel].reshape(-1)
    want = O.block_gemm(payload, ob, sel.size, cols, X, wide=True)
    assert rel_l2(y[:, sel], want) <= TOL


def test_shape_errors():
    w = gaussian_weights(256 * 3 + 10, 1)
    payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL4)
    with ia.DeviceWeights.from_blocks(payload, blocks, 1, w.size) as dw:
        with pytest.raises(ia.OilHipError):
            dw.gemv(torch.zeros(1, w.size, device="cuda"))        # ragged block: matmul refuses


# The multi-row kernel splits activations into two FP16 parts after scaling each token row by a power of two, so its
# accuracy must not depend on the magnitude of the activations: tiny rows, huge rows (beyond the FP16 range), rows that
# mix magnitudes, a zero row, and tokens of very different scale in one batch.
@pytest.mark.parametrize("rows,cols,M", [(130, 4096, 5), (61, 11008, 16), (300, 2048, 24)])
def test_oil4_multi_token_activation_ranges(rows, cols, M):
    w = gaussian_weights(rows * cols, rows + cols)
    payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL4)
    rng = np.random.default_rng(M)
    X = rng.standard_normal((M, cols)).astype(np.float32)
    X[0] *= np.float32(1e-6)
    X[1] *= np.float32(1e5)
    X[2] *= np.float32(3e-30)
    X[3] *= np.float32(2e30)
    X[4, ::3] *= np.float32(1e-7)                         # one row with magnitudes 14 decades apart
    X[4, 1::3] *= np.float32(1e7)
    if M > 5:
        X[5] = 0.0
    want = O.block_gemm(payload, to_orc_blocks(blocks), rows, cols, X, wide=True)
    with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
        got = dw.gemv(torch.from_numpy(X).cuda()).cpu().numpy()
    for m in range(M):                                    # row by row: a large row must not hide a small one
        assert rel_l2(got[m], want[m]) <= TOL, m


def test_two_streams_run_multi_token_gemvs_concurrently():
    """Calls on different streams keep separate activation scratch: M = 16 GEMVs of two tensors issued back and forth
    on two streams, all in flight together, the first and last round checked against the oracle, one in between
    against a quiet rerun."""
    shapes = [(2048, 4096), (1024, 11008)]
    rng = np.random.default_rng(21)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    handles, wants, outs, xs = [], [], [], []
    rounds = 12
    for i, (rows, cols) in enumerate(shapes):
        w = gaussian_weights(rows * cols, 50 + i)
        payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL4)
        handles.append(ia.DeviceWeights.from_blocks(payload, blocks, rows, cols))
        X = rng.standard_normal((rounds, 16, cols)).astype(np.float32)
        xs.append(torch.from_numpy(X).cuda())
        wants.append([O.block_gemm(payload, to_orc_blocks(blocks), rows, cols, X[r], wide=True) for r in (0, rounds - 1)])
        outs.append([None] * rounds)
    torch.cuda.synchronize()
    for r in range(rounds):
        for i in (0, 1):
            with torch.cuda.stream(streams[i]):
                outs[i][r] = handles[i].gemv(xs[i][r])
    torch.cuda.synchronize()
    for i in (0, 1):
        for r, want in zip((0, rounds - 1), wants[i]):
            assert rel_l2(outs[i][r].cpu().numpy(), want) <= TOL, (i, r)
        # the rounds in between: same weights, so linear in the activations
        mid = outs[i][5].cpu().numpy()
        with torch.cuda.stream(streams[i]):
            again = handles[i].gemv(xs[i][5])
        streams[i].synchronize()
        assert np.array_equal(mid, again.cpu().numpy()), i
    for h in handles:
        h.close()


def test_release_stream_scratch_frees_every_buffer_of_the_stream():
    """A stream's scratch grows with the requests (the smaller buffer is kept for graphs that may point at it);
    oilhip_release_stream_scratch returns all of it, and the next call on the stream allocates afresh and agrees."""
    st = torch.cuda.Stream()
    rng = np.random.default_rng(31)
    cases = []
    for rows, cols, M in ((256, 4096, 5), (8192, 11008, 16)):       # packed activations (4 MB), then partial sums on top
        w = gaussian_weights(rows * cols, rows + M)
        payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL4)
        cases.append((ia.DeviceWeights.from_blocks(payload, blocks, rows, cols),
                      torch.from_numpy(rng.standard_normal((M, cols)).astype(np.float32)).cuda(),
                      torch.empty(M, rows, device="cuda"), torch.empty(M, rows, device="cuda")))
    release = ia._lib.lib().oilhip_release_stream_scratch
    with torch.cuda.stream(st):
        cases[0][3].zero_()                                          # the runtime sets up the stream's queue on its first launch
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    with torch.cuda.stream(st):
        for dw, x, y, _ in cases:
            dw.gemv(x, out=y)
    st.synchronize()
    held = free0 - torch.cuda.mem_get_info()[0]
    assert held >= 12 << 20                                          # the first buffer and the one that replaced it
    ia._lib.check(release(st.cuda_stream))
    assert torch.cuda.mem_get_info()[0] >= free0
    with torch.cuda.stream(st):
        for dw, x, _, y2 in cases:
            dw.gemv(x, out=y2)
    st.synchronize()
    for dw, x, y, y2 in cases:
        assert np.array_equal(y.cpu().numpy(), y2.cpu().numpy())
    ia._lib.check(release(st.cuda_stream))
    for dw, *_ in cases:
        dw.close()
