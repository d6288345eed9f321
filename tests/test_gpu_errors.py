"""Error behaviour of the C ABI on the GPU: bad arguments come back as status codes with a message
(which the Python layer raises as RuntimeError, the reference's exception type), and no kernel runs."""
import ctypes as C

import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_weight_kn, make_x

pytestmark = pytest.mark.gpu

CI_ERR_ARG, CI_ERR_CAPACITY = 1, 3


def _t32(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int32))


def _dev_enc(oracle, K, N, th=1024, tw=32, seed=5):
    w = make_weight_kn(N, K, seed=seed)
    enc, man = oracle.compress_bf16(bf16_bits(w), th, tw)
    d = "cuda"
    return dict(stream=torch.from_numpy(enc.stream).to(d), states=_t32(enc.states).to(d),
                tables=_t32(enc.tables).to(d), slot_map=torch.from_numpy(enc.slot_map).to(d),
                offs=_t32(enc.tile_offsets).to(d), lens=_t32(enc.tile_max_lens).to(d),
                man=torch.from_numpy(man).to(d).view(-1)), w


def _p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p()


def test_device_check_passes_on_this_gpu():
    from comp_inference_amd import _lib

    assert _lib.lib().ci_check_device() == 0


def test_linear_workspace_too_small_is_a_capacity_error(oracle):
    from comp_inference_amd import _lib

    K, N, M = 14336, 64, 2  # 14 k-tiles: two partial sums need a workspace
    e, _ = _dev_enc(oracle, K, N)
    x = make_x(M, K, seed=1).cuda()
    out = torch.full((M, N), 3.0, dtype=torch.bfloat16, device="cuda")
    lib = _lib.lib()
    need = lib.ci_fused_linear_workspace_bytes(M, K, N, 1024, 32, 0)
    assert need >= 2 * M * N * 4
    rc = lib.ci_fused_linear_ilp2(_p(x), M, K, N, K, _p(e["stream"]), C.c_uint64(e["stream"].numel()), _p(e["states"]),
                                  _p(e["tables"]), _p(e["slot_map"]), _p(e["offs"]), _p(e["lens"]), _p(e["man"]), 1024,
                                  32, None, _p(out), N, None, C.c_size_t(0), None)
    assert rc == CI_ERR_CAPACITY and b"workspace" in lib.ci_last_error()
    torch.cuda.synchronize()
    assert torch.all(out == 3.0)  # nothing ran


def test_null_and_misshapen_arguments_are_rejected(oracle):
    from comp_inference_amd import _lib

    K, N = 1024, 64
    e, _ = _dev_enc(oracle, K, N)
    out = torch.empty((K, N), dtype=torch.uint8, device="cuda")
    lib = _lib.lib()
    args = lambda **kw: (  # noqa: E731
        _p(kw.get("stream", e["stream"])), C.c_uint64(e["stream"].numel()), _p(kw.get("states", e["states"])),
        _p(e["tables"]), _p(e["slot_map"]), _p(e["offs"]), _p(e["lens"]), K, N, kw.get("th", 1024), 32,
        _p(kw.get("out", out)), None, None, None)
    assert lib.ci_decode_tiled_ilp2(*args()) == 0
    assert lib.ci_decode_tiled_ilp2(*args(states=None)) == CI_ERR_ARG
    assert lib.ci_decode_tiled_ilp2(*args(out=None)) == CI_ERR_ARG
    assert lib.ci_decode_tiled_ilp2(*args(th=1023)) == CI_ERR_ARG  # odd tile height
    assert lib.ci_last_error() != b""
    seg = lambda ck, segs: args()[:11] + (_p(ck), segs) + args()[11:]  # noqa: E731
    ck = torch.zeros(lib.ci_checkpoint_bytes(K, N, 1024, 32, 4) // 8, dtype=torch.int64, device="cuda")
    assert lib.ci_decode_tiled_ilp2_segmented(*seg(None, 4)) == CI_ERR_ARG     # segments without checkpoints
    assert lib.ci_decode_tiled_ilp2_segmented(*seg(ck, 3)) == CI_ERR_ARG       # 512 rows do not split in 3 x 16 n
    assert lib.ci_decode_tiled_ilp2_segmented(*seg(None, 1)) == 0
    x = make_x(1, K, seed=1).cuda()
    o = torch.empty((1, N), dtype=torch.bfloat16, device="cuda")
    rc = lib.ci_fused_linear_ilp2(_p(x), 1, K, N, K - 8, _p(e["stream"]), C.c_uint64(e["stream"].numel()),
                                  _p(e["states"]), _p(e["tables"]), _p(e["slot_map"]), _p(e["offs"]), _p(e["lens"]),
                                  _p(e["man"]), 1024, 32, None, _p(o), N, None, C.c_size_t(0), None)
    assert rc == CI_ERR_ARG  # row stride shorter than the row
    torch.cuda.synchronize()


def test_python_layer_raises_runtime_error(oracle):
    from comp_inference_amd import fused_rans_linear

    K, N = 1024, 64
    e, _ = _dev_enc(oracle, K, N)
    x = make_x(1, K, seed=1).cuda()
    odd = torch.zeros(4097, dtype=torch.uint8, device="cuda")[1:]      # 4096 entries at an odd address
    odd.copy_(e["slot_map"])
    with pytest.raises(RuntimeError, match="slot_map"):                 # the library's message, raised in Python
        fused_rans_linear(x, e["stream"], e["states"], e["tables"], odd, (K, N), e["offs"], e["lens"], 1024, 32, e["man"])
    with pytest.raises(ValueError, match="size mismatch"):              # operand lengths are checked before that
        fused_rans_linear(x, e["stream"], e["states"], e["tables"], e["slot_map"], (K, N), e["offs"], e["lens"], 1023, 32,
                          e["man"])


def test_stream_shorter_than_the_offsets_claim_decodes_without_reading_past_it(oracle):
    """A truncated stream must not be read beyond its length: tiles whose body would run past the
    end are treated as empty (their symbols are then wrong, but nothing outside the buffer is touched)."""
    from comp_inference_amd import rans_decomp_tiled

    K, N = 2048, 64
    e, _ = _dev_enc(oracle, K, N)
    short = e["stream"][: e["stream"].numel() // 2].clone()
    out = rans_decomp_tiled(short, e["states"], e["tables"], e["slot_map"], (K, N), e["offs"], e["lens"], tile_k=1024,
                            tile_n=32)
    torch.cuda.synchronize()
    assert out.shape == (K, N)
