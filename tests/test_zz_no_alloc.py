"""The entry point that allocates nothing (ci_fused_linear_tiled_noalloc) against the entry point that takes a
workspace (ci_fused_linear_tiled), through the C ABI: the same kernels in the same order, so the outputs are
compared bit for bit; and against torch.matmul on the oracle-decoded weight within the operator's tolerance.
Two calls in a row share the library's scratch array, the second with a smaller input."""
import ctypes as C

import numpy as np
import pytest
import torch

from helpers import bf16_bits, bits_to_bf16, make_weight_kn, make_x

pytestmark = pytest.mark.gpu
ATOL = RTOL = 1e-2


def _t32(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int32))


class _Weight:
    def __init__(self, oracle, K, N, th, segments, seed):
        import comp_inference_amd as ci
        from comp_inference_amd import _lib

        dev = torch.device("cuda", 0)
        w = make_weight_kn(N, K, seed=seed)
        enc, man = oracle.compress_bf16(bf16_bits(w), th, 32)
        self.wdec = bits_to_bf16(oracle.decompress_bf16(enc, man, K, N))
        self.K, self.N, self.th, self.segments = K, N, th, segments
        self.t = [torch.from_numpy(enc.stream).to(dev), _t32(enc.states).to(dev), _t32(enc.tables).to(dev),
                  torch.from_numpy(enc.slot_map).to(dev), _t32(enc.tile_offsets).to(dev),
                  _t32(enc.tile_max_lens).to(dev), torch.from_numpy(man).to(dev)]
        self.ck = None
        if segments > 1:
            self.ck = ci.build_checkpoints(self.t[0], self.t[1], self.t[2], self.t[3], (K, N), self.t[4], self.t[5],
                                           th, 32, segments)
        t = self.t
        self.desc = _lib.tiled_weight(K, N, th, 32, t[0], t[1], t[2], t[3], t[4], t[5], t[6], self.ck, segments)


def _both(wt, x):
    """(output of the no-allocation entry point, output of the workspace entry point) for x [M, K] on the GPU."""
    from comp_inference_amd import _lib

    lib, ptr = _lib.lib(), _lib.ptr
    M = x.shape[0]
    need = lib.ci_fused_linear_workspace_bytes_segmented(M, wt.K, wt.N, wt.th, 32, 0, wt.segments)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=x.device)
    out_ws = torch.full((M, wt.N), 7.0, dtype=torch.bfloat16, device=x.device)
    out_na = torch.full((M, wt.N), -7.0, dtype=torch.bfloat16, device=x.device)
    stream = _lib.stream_handle(x.device)
    _lib.check(lib.ci_fused_linear_tiled(C.byref(wt.desc), ptr(x), M, x.stride(0), None, ptr(out_ws), wt.N, ptr(ws),
                                         C.c_size_t(ws.numel()), stream))
    # nothing below allocates: every tensor exists already
    before = torch.cuda.memory_allocated(x.device)
    _lib.check(lib.ci_fused_linear_tiled_noalloc(C.byref(wt.desc), ptr(x), M, x.stride(0), None, ptr(out_na), wt.N,
                                                 stream))
    assert torch.cuda.memory_allocated(x.device) == before
    torch.cuda.synchronize()
    return out_na, out_ws


def test_two_calls_in_a_row_share_the_scratch_array(oracle):
    """A 14-tile-row weight (partial sums through the scratch array and the reduction kernel) at 40 rows of x
    (the fragment copy of x lives in the scratch array too), then a smaller weight at 3 rows."""
    big = _Weight(oracle, 14336, 96, 1024, 2, seed=11)
    small = _Weight(oracle, 3072, 64, 512, 1, seed=12)
    dev = torch.device("cuda", 0)
    for wt, M, seed in ((big, 40, 1), (small, 3, 2), (big, 1, 3)):
        x = make_x(M, wt.K, seed=seed).to(dev)
        got, same = _both(wt, x)
        assert torch.equal(got.view(torch.int16), same.view(torch.int16))
        want = torch.matmul(x.float().cpu(), wt.wdec.float())
        assert torch.allclose(got.float().cpu(), want, atol=ATOL, rtol=RTOL), (got.float().cpu() - want).abs().max()


def test_a_shape_beyond_the_scratch_array_is_refused(oracle):
    from comp_inference_amd import _lib

    wt = _Weight(oracle, 1024, 64, 1024, 1, seed=13)
    lib = _lib.lib()
    desc = wt.desc
    # the same arrays described as a weight so tall that its partial sums cannot fit: refused on the host, before
    # any array is touched (the length checks of the descriptor come first, so the lengths are made to agree)
    K = 1024 * 4096
    desc.K = K
    desc.n_states = desc.n_tiles = desc.man_len = 1 << 40
    x = torch.zeros(64, 8, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(64, wt.N, dtype=torch.bfloat16, device="cuda")
    need = lib.ci_fused_linear_workspace_bytes_segmented(64, K, wt.N, 1024, 32, 0, 1)
    assert need > 16 << 20
    rc = lib.ci_fused_linear_tiled_noalloc(C.byref(desc), _lib.ptr(x), 64, K, None, _lib.ptr(out), wt.N, None)
    assert rc == 3  # CI_ERR_CAPACITY
    assert b"scratch" in lib.ci_last_error()
