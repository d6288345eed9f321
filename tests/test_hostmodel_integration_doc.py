"""The ctypes binding that the integration notes at the repository root give a maintainer of the reference to copy,
taken from the file as it stands and run (on the host model): the two functions it defines must agree with the package's own operators on a
compressed weight, so the argument order and types printed there are the library's."""
import os
import re

from tests.hostmodel.model import in_fresh_process

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@in_fresh_process
def test_the_binding_printed_in_the_integration_notes_runs():
    import torch

    from tests.hostmodel.backend import python_api_on_hostmodel

    notes = next(f for f in sorted(os.listdir(ROOT)) if f.upper().startswith("INTEGRATION") and f.endswith(".md"))
    text = open(os.path.join(ROOT, notes)).read()
    blocks = re.findall(r"```python\n(.*?)```", text, flags=re.S)
    (code,) = [b for b in blocks if "_hip_backend.py" in b]
    assert 'C.CDLL("libcomp_inference_hip.so")' in code
    with python_api_on_hostmodel():
        import comp_inference_amd as ci
        from comp_inference_amd import _lib

        ns = {}
        exec(code.replace('"libcomp_inference_hip.so"', repr(_lib.LIB_PATH)), ns)  # the host-model build of the same ABI
        torch.manual_seed(3)
        K, N, th = 1024, 80, 512
        w = (torch.randn(K, N) * 0.02).to(torch.bfloat16)
        exp, man = ci.extract_exp_and_mantissa(w)
        f, c = ci.get_rans_lut(exp)
        r = ci.ccore.RansManager(exp.numel()).compress_tiled(exp, f, c, th, 32)
        man_t = ci.interleave_mantissas(man, th, 32)
        ops = (r.stream, r.states, r.tables, r.slot_map, (K, N), r.tile_offsets, r.tile_max_lens)
        got = ns["rans_decomp_triton_tiled"](*ops, tile_k=th, tile_n=32)
        assert got.dtype == torch.uint8 and torch.equal(got, exp)
        bias = (torch.randn(N) * 0.1).to(torch.bfloat16)
        for shape in ((1, K), (5, K), (2, 3, K)):
            x = torch.randn(*shape).to(torch.bfloat16)
            y = ns["fused_rans_linear_triton"](x, *ops, th, 32, man_t, bias=bias)
            want = ci.fused_rans_linear_triton(x, *ops, th, 32, man_t, bias=bias)
            assert y.shape == (*shape[:-1], N) and torch.equal(y.view(torch.int16), want.view(torch.int16))
            ref = x.float().reshape(-1, K) @ w.float() + bias.float()
            assert torch.allclose(y.float().reshape(-1, N), ref, atol=1e-2, rtol=1e-2)
