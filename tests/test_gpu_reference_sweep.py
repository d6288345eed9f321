"""The reference's main parity script as a test (tests/test_mat_mul.py:108-259, sweep :263-264):
K, N = 3072, 1024, x of 8192 rows, weights torch.randn bf16, every tile height in 32..1024 and tile
width in 16..128; the fused result and (stand-alone decode -> reassemble -> torch.matmul) against
torch.matmul(x, W) with allclose(atol=1e-2, rtol=1e-2) on the bf16 results, through the entry points
and argument names the script uses."""
import pytest
import torch

pytestmark = pytest.mark.gpu

HEIGHTS = [32, 64, 128, 256, 512, 1024]
WIDTHS = [16, 32, 64, 128]
K, N = 3072, 1024


def _module(weights_kn, tile_height, tile_width):
    from comp_inference_amd import rans_compress_module_weight

    module = torch.nn.Module()
    module.weight = torch.nn.Parameter(weights_kn.clone().contiguous())
    module.bias = None
    rans_compress_module_weight(module, tile_height=tile_height, tile_width=tile_width, transpose_weight=False)
    return module


def _fused(module, x, tile_height, tile_width):
    from comp_inference_amd import fused_rans_linear_triton

    return fused_rans_linear_triton(
        x=x,
        compressed_data=module.exponent_compressed_weight.cuda(),
        initial_states=module.exponent_states.cuda(),
        tables=module.exponent_tables.cuda(),
        slot_map=module.exponent_slot_map.cuda(),
        weight_shape=(K, N),
        tile_offsets=module.exponent_tile_offsets.cuda(),
        tile_max_lens=module.exponent_tile_max_lens.cuda(),
        tile_k=tile_height,
        tile_n=tile_width,
        mantissas=module.mantissa_raw.cuda(),
        bias=module.bias,
        accum_block_size=tile_width,
    )


@pytest.fixture(scope="module")
def data():
    g = torch.Generator("cuda").manual_seed(1234)
    weights_kn = torch.randn((K, N), dtype=torch.bfloat16, device="cuda", generator=g)
    x = torch.randn((8192, K), dtype=torch.bfloat16, device="cuda", generator=g)
    return weights_kn, x, torch.matmul(x, weights_kn)


@pytest.mark.parametrize("tile_width", WIDTHS)
@pytest.mark.parametrize("tile_height", HEIGHTS)
def test_module_integration(data, tile_height, tile_width):
    from comp_inference_amd import rans_decomp_triton_tiled, reconstruct_from_exp_and_mantissa, uninterleave_mantissas

    weights_kn, x, result_golden = data
    module = _module(weights_kn, tile_height, tile_width)

    result_compressed = _fused(module, x, tile_height, tile_width)

    decomp_exp = rans_decomp_triton_tiled(
        compressed_streams=module.exponent_compressed_weight.cuda(),
        initial_states=module.exponent_states.cuda(),
        tables=module.exponent_tables.cuda(),
        slot_map=module.exponent_slot_map.cuda(),
        output_shape=(K, N),
        tile_offsets=module.exponent_tile_offsets.cuda(),
        tile_max_lens=module.exponent_tile_max_lens.cuda(),
        tile_k=tile_height,
        tile_n=tile_width,
    )
    decomp_man = uninterleave_mantissas(module.mantissa_raw.cuda(), K, N, TILE_K=tile_height, TILE_N=tile_width)
    reassembled_weight = reconstruct_from_exp_and_mantissa(decomp_exp, decomp_man, dtype=torch.bfloat16)
    # stricter than the script: the weight comes back bit for bit
    assert torch.equal(reassembled_weight.view(torch.int16), weights_kn.view(torch.int16))
    result_decomp = torch.matmul(x, reassembled_weight)

    assert result_golden.shape == result_compressed.shape == result_decomp.shape
    assert torch.allclose(result_golden, result_compressed, atol=1e-2, rtol=1e-2), \
        (result_golden - result_compressed).abs().max()
    assert torch.allclose(result_golden, result_decomp, atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("tile_width", WIDTHS)
@pytest.mark.parametrize("tile_height", HEIGHTS)
def test_module_integration_on_the_fused_kernels(data, always_fused, tile_height, tile_width):
    """The same sweep with the weight decoded inside the product (128 rows of x: two passes of the
    32-column kernel, sixteen of the any-width kernel)."""
    weights_kn, x, result_golden = data
    module = _module(weights_kn, tile_height, tile_width)
    result_compressed = _fused(module, x[:128], tile_height, tile_width)
    assert torch.allclose(result_golden[:128], result_compressed, atol=1e-2, rtol=1e-2), \
        (result_golden[:128] - result_compressed).abs().max()


@pytest.mark.parametrize("Kw,Nw", [(4096, 1024), (1024, 4096)])
def test_split_k_sweep(Kw, Nw):
    """The reference's SPLIT_K sweep (tests/test_split_k.py:94-230) with its own call pattern: both tiled
    layouts, batch sizes 1-64, SPLIT_K 1-16, stream sizes of the one-stream-per-column layout taken as
    successive differences of the offsets (:142-147).  The reference only times these calls; here the
    result must not depend on SPLIT_K at all (partitioning is chosen from the shape) and must meet the
    allclose(1e-2, 1e-2) bar against torch.matmul."""
    from comp_inference_amd import (fused_rans_linear_triton, fused_rans_linear_triton_uncoalesced,
                                    rans_compress_module_weight)

    g = torch.Generator("cuda").manual_seed(Kw)
    weights_kn = (torch.randn((Kw, Nw), device="cuda", generator=g) * 0.02).to(torch.bfloat16)
    mods = {}
    for uncoalesced in (False, True):
        mod = torch.nn.Module()
        mod.weight = torch.nn.Parameter(weights_kn.clone())
        mod.bias = None
        rans_compress_module_weight(mod, tile_height=1024, tile_width=32, transpose_weight=False,
                                    uncoalesced_interleaving=uncoalesced)
        mods[uncoalesced] = mod
    c, u = mods[False], mods[True]
    u_off = u.exponent_stream_offsets.cuda()
    u_tot = torch.tensor([u.exponent_compressed_weight.numel()], dtype=torch.int64, device="cuda")
    u_sizes = (torch.cat([u_off.to(torch.int64)[1:], u_tot]) - u_off.to(torch.int64)).to(torch.uint32)
    for bs in (1, 8, 64):
        x = torch.randn((bs, Kw), dtype=torch.bfloat16, device="cuda", generator=g)
        want = torch.matmul(x, weights_kn).float()
        first = {}
        for sk in (1, 2, 4, 8, 16):
            coal = fused_rans_linear_triton(
                x=x, compressed_data=c.exponent_compressed_weight.cuda(), initial_states=c.exponent_states.cuda(),
                tables=c.exponent_tables.cuda(), slot_map=c.exponent_slot_map.cuda(), weight_shape=(Kw, Nw),
                tile_offsets=c.exponent_tile_offsets.cuda(), tile_max_lens=c.exponent_tile_max_lens.cuda(),
                tile_k=1024, tile_n=32, mantissas=c.mantissa_raw.cuda(), accum_block_size=32, SPLIT_K=sk)
            unco = fused_rans_linear_triton_uncoalesced(
                x=x, compressed_data=u.exponent_compressed_weight.cuda(), initial_states=u.exponent_states.cuda(),
                tables=u.exponent_tables.cuda(), slot_map=u.exponent_slot_map.cuda(), weight_shape=(Kw, Nw),
                stream_offsets=u_off, stream_sizes=u_sizes, tile_k=1024, tile_n=32, mantissas=u.mantissa_raw.cuda(),
                accum_block_size=32, SPLIT_K=sk)
            for name, got in (("coalesced", coal), ("uncoalesced", unco)):
                assert torch.allclose(got.float(), want, atol=1e-2, rtol=1e-2), (name, bs, sk)
                ref = first.setdefault(name, got)
                assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), (name, bs, sk)
