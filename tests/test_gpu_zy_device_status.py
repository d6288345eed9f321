"""The fused linear's one wait between wavefronts is bounded, and a wait that gives up is reported (not a GPU hang)."""
import numpy as np
import pytest
import torch

import comp_inference_amd as ci
from tests.helpers import make_weight_kn, make_x

pytestmark = pytest.mark.gpu


def _prepared(K, N, th, segs, dev):
    w = make_weight_kn(N, K, 1)
    exp, man = ci.extract_exp_and_mantissa(w)
    f, c = ci.get_rans_lut(exp)
    res = ci.ccore.RansManager(exp.numel()).compress_tiled(exp, f, c, th, 32)
    man_t = ci.interleave_mantissas(man, th, 32)
    args = [t.to(dev) for t in (res.stream, res.states, res.tables, res.slot_map)]
    offs, lens = res.tile_offsets.to(dev), res.tile_max_lens.to(dev)
    ck = ci.build_checkpoints(args[0], args[1], args[2], args[3], (K, N), offs, lens, th, 32, segs)
    return w, (args, offs, lens, man_t.to(dev), ck)


def test_forced_give_up_ends_the_kernel_and_is_reported():
    """The number of looks forced to zero from the host: every wait gives up without looking at its flag, whoever
    got where first.  The kernel
    ends all the same, ci_device_status says what happened once and is clear afterwards; with the default limit
    the same launches leave the status word clear and give the usual sums."""
    dev = torch.device("cuda", 0)
    K, N, th, segs = 768, 20000, 256, 2  # 625 column tiles, 6 items each: several jobs per workgroup
    w, (args, offs, lens, man, ck) = _prepared(K, N, th, segs, dev)
    x = make_x(2, K, 2).to(dev)

    def run():
        return ci.fused_rans_linear(x, args[0], args[1], args[2], args[3], (K, N), offs, lens, th, 32, man,
                                    checkpoints=ck, segments=segs)

    want = (x.float() @ w.to(dev).float())
    y = run()
    assert ci.device_status(dev) == 0
    assert torch.allclose(y.float(), want, atol=1e-2, rtol=1e-2)
    before = ci.debug_wait_limit(0)
    try:
        run()  # whatever it computes: the point is that it ends
        torch.cuda.synchronize()
        with pytest.raises(RuntimeError, match="bounded wait"):
            ci.device_status(dev)
        assert ci.device_status(dev) == 0
    finally:
        ci.debug_wait_limit(before)
    y2 = run()
    assert ci.device_status(dev) == 0 and torch.equal(y2, y)
