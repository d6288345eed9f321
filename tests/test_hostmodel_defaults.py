"""Which kernels the runtime modules launch as they come, and with each switch turned on (host model: the launch
list is the library's own).  The kernels that have not run on a GPU yet sit behind switches that are off by default:
a module used as the reference's is used must not reach them, and each switch must reach what it names."""
import numpy as np
import pytest
import torch
import torch.nn as nn

from tests.hostmodel.model import in_child

NOT_YET_ON_A_GPU = ("embed_gather32_seg_kernel", "trans32_seg_kernel", "fused_linear32_wide_kernel")


def _launches(lib):
    names = [lib.sim_launch_name(i).decode() for i in range(lib.sim_launch_count())]
    lib.sim_clear()
    return names


def _modules():
    import comp_inference_amd as ci

    torch.manual_seed(3)
    lin = nn.Linear(2048, 96, bias=True).to(torch.bfloat16)
    emb = nn.Embedding(2048, 64).to(torch.bfloat16)
    head = nn.Linear(64, 2048, bias=False).to(torch.bfloat16)
    with torch.no_grad():
        for m in (lin, emb, head):
            m.weight.mul_(0.05)
    keep = dict(lin=lin.weight.detach().clone(), bias=lin.bias.detach().clone(), emb=emb.weight.detach().clone(),
                head=head.weight.detach().clone())
    ci.rans_compress_module_weight(lin, tile_height=1024, tile_width=32)
    ci.rans_compress_module_weight(emb, tile_height=1024, tile_width=32, transpose_weight=False)
    ci.rans_compress_module_weight(head, tile_height=1024, tile_width=32, transpose_weight=False)
    return (ci.RansLinear.from_compressed(lin, bias=keep["bias"]), ci.RansEmbedding.from_compressed(emb),
            ci.RansLMHead.from_compressed(head) if hasattr(ci.RansLMHead, "from_compressed") else None, keep)


@in_child
def test_modules_as_they_come_and_with_each_switch_on():
    import ctypes as C

    import comp_inference_amd as ci
    from comp_inference_amd import _lib
    from tests.hostmodel.backend import python_api_on_hostmodel

    with python_api_on_hostmodel(cus=4):
        lib = _lib.lib()
        lib.sim_launch_name.restype = C.c_char_p
        rl, re_, rh, keep = _modules()
        if rh is None:
            rh = ci.RansLMHead(64, 2048)
            src = nn.Linear(64, 2048, bias=False).to(torch.bfloat16)
            src.weight.data = keep["head"].clone()
            ci.rans_compress_module_weight(src, tile_height=1024, tile_width=32, transpose_weight=False)
            from comp_inference_amd.pytorch_runtime import _load_from_compressed

            _load_from_compressed(rh, src)
        ids = torch.tensor([0, 5, 2047, 1024, 5])
        x1, x40, x100 = (torch.randn(m, 2048).to(torch.bfloat16) for m in (1, 40, 100))
        h1, h3 = torch.randn(1, 64).to(torch.bfloat16), torch.randn(3, 64).to(torch.bfloat16)

        def check_all():
            for x in (x1, x40, x100):
                want = x.float() @ keep["lin"].float().t() + keep["bias"].float()
                assert torch.allclose(rl(x.cuda()).float().cpu(), want, atol=2e-2, rtol=2e-2)
            assert torch.equal(re_(ids.cuda()).cpu().view(torch.int16), keep["emb"][ids].view(torch.int16))
            for h in (h1, h3):
                assert torch.allclose(rh(h.cuda()).float().cpu(), h.float() @ keep["head"].float().t(), atol=2e-2, rtol=2e-2)

        lib.sim_clear()
        check_all()
        default = _launches(lib)
        assert not [k for k in default if any(n in k for n in NOT_YET_ON_A_GPU)], default
        # what the defaults are: checkpoints for the linear and the table, the sixteen-wavefront fused linear, the
        # whole-tile gather and head, and above 64 rows one merged decode for the library GEMM
        for name in ("checkpoints_kernel", "fused_linear32_seg_kernel<1, false>", "fused_linear32_seg_kernel<2, false>",
                     "embed_gather32_kernel", "trans32_kernel<1>", "trans32_kernel<kTrRows>"):
            assert any(name in k for k in default), (name, default)
        assert any("decode_tiled32" in k and "true" in k for k in default), default  # the merged decode for 100 rows

        # each switch reaches the kernel it names, with the same results
        re_.sixteen_wavefronts = True
        rh.segments = 4
        before = ci.fused_wide_rows(True)
        try:
            from comp_inference_amd import linear_hip

            saved, linear_hip.DECODE_ONCE_ABOVE_ROWS = linear_hip.DECODE_ONCE_ABOVE_ROWS, None
            try:
                check_all()
            finally:
                linear_hip.DECODE_ONCE_ABOVE_ROWS = saved
        finally:
            ci.fused_wide_rows(before)
        switched = _launches(lib)
        for name in NOT_YET_ON_A_GPU:
            assert any(name in k for k in switched), (name, switched)
        ci.head_matrix_sums(True)
        try:
            assert torch.allclose(rh(h1.cuda()).float().cpu(), h1.float() @ keep["head"].float().t(), atol=2e-2, rtol=2e-2)
        finally:
            ci.head_matrix_sums(False)
        assert any("trans32_seg_kernel<true>" in k for k in _launches(lib))
