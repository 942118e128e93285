"""oilhip_gemv_oil4_f32_noalloc (the entry point that allocates no device memory: its scratch is a fixed device array)
against oilhip_gemv_f32 on the same inputs, through the C ABI, on two calls in a row of which the second is smaller.

Bars: both entry points run the same kernels, so outputs are compared bit for bit where the kernel's sum order is
fixed (rows of at most 4096 weights, or fewer than three activation rows) and within relative L2 1e-5 otherwise, and
both are checked against the oracle's double-precision sums at 1e-5."""
import numpy as np
import pytest
import torch

import innova_amd as ia
import oracle as O
from gpu_util import gaussian_weights, rel_l2, to_orc_blocks

pytestmark = pytest.mark.gpu
TOL = 1e-5


def both(dw, X):
    xd = torch.from_numpy(X).cuda()
    want = dw.gemv(xd).cpu().numpy()
    got = dw.gemv(xd, noalloc=True).cpu().numpy()
    return got, want


@pytest.mark.parametrize("first,second", [((300, 4096, 16), (130, 2048, 5)),       # one K-pass: fixed sum order
                                          ((200, 11008, 24), (64, 4096, 3)),       # rows cut along K, passes of 32 and 8
                                          ((96, 4096, 2), (50, 768, 1))])          # the register kernel: no scratch at all
def test_noalloc_matches_gemv(first, second):
    for rows, cols, M in (first, second):                  # the second call finds the first call's bytes in the scratch
        w = gaussian_weights(rows * cols, rows + cols + M)
        payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL4)
        X = np.random.default_rng(M + rows).standard_normal((M, cols)).astype(np.float32)
        with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
            got, want = both(dw, X)
        if cols <= 4096 or M <= 2:
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        assert rel_l2(got, want) <= TOL
        ref = O.block_gemm(payload, to_orc_blocks(blocks), rows, cols, X, wide=True)
        assert rel_l2(got, ref) <= TOL


def test_noalloc_allocates_nothing_and_runs_under_capture_on_a_fresh_stream():
    """A shape whose kernel needs scratch (five rows, 11008 columns: packed activations, three K parts that meet in
    the scratch): the call leaves the device's free memory as it found it on a stream the library has never seen, and
    the same call is captured into a graph on another fresh stream (where a scratch allocation would be refused) and
    replayed."""
    rows, cols, M = 200, 11008, 5
    w = gaussian_weights(rows * cols, 77)
    payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL4)
    X = np.random.default_rng(78).standard_normal((M, cols)).astype(np.float32)
    with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
        x = torch.from_numpy(X).cuda()
        want = dw.gemv(x).clone()
        y = torch.zeros(M, rows, device="cuda")
        dw.gemv(x, out=y, noalloc=True)                   # the library's code object and the scratch address are in place
        torch.cuda.synchronize()
        st = torch.cuda.Stream()
        with torch.cuda.stream(st):
            y.zero_()                                     # the runtime sets up the stream's queue on its first launch
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        with torch.cuda.stream(st):
            dw.gemv(x, out=y, noalloc=True)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free0
        assert rel_l2(y.cpu().numpy(), want.cpu().numpy()) <= TOL
        st2 = torch.cuda.Stream()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(st2):
            y.zero_()
            st2.synchronize()
            with torch.cuda.graph(g, stream=st2):
                dw.gemv(x, out=y, noalloc=True)
            for _ in range(3):
                y.zero_()
                g.replay()
                st2.synchronize()
                assert rel_l2(y.cpu().numpy(), want.cpu().numpy()) <= TOL
    ref = O.block_gemm(payload, to_orc_blocks(blocks), rows, cols, X, wide=True)
    assert rel_l2(want.cpu().numpy(), ref) <= TOL


def test_noalloc_refuses_partial_sums_beyond_the_scratch():
    rows, cols, M = 24000, 11008, 16                                  # 3 parts x 16 tokens x 24000 rows > 1,043,456 floats
    payload = np.zeros(rows * cols // 2, dtype=np.uint8)
    blocks = np.zeros(rows * cols // 256, dtype=ia._lib.BLOCK_DTYPE)
    blocks["idx_off"] = np.arange(blocks.size, dtype=np.uint64) * 128
    blocks["cb_off"] = blocks["idx_off"]
    blocks["idx_bytes"], blocks["nw"], blocks["fmt"] = 128, 256, int(ia.Format.OIL4)
    with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
        x = torch.zeros(M, cols, device="cuda")
        with pytest.raises(ia.OilHipError, match="needs a kernel that allocates"):
            dw.gemv(x, noalloc=True)
        assert torch.count_nonzero(dw.gemv(x)).item() == 0           # the allocating entry point takes the shape


def test_noalloc_rejects_what_it_cannot_serve():
    w = gaussian_weights(8 * 512, 3)
    payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL8)
    with ia.DeviceWeights.from_blocks(payload, blocks, 8, 512) as dw:
        with pytest.raises(ia.OilHipError, match="uniform OIL4"):
            dw.gemv(torch.zeros(1, 512, device="cuda"), noalloc=True)
    rows, cols = 4, 32768 + 256                                       # wider than the fixed scratch
    w = gaussian_weights(rows * cols, 4)
    payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL4)
    with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
        with pytest.raises(ia.OilHipError, match="exceed the static scratch"):
            dw.gemv(torch.zeros(5, cols, device="cuda"), noalloc=True)
