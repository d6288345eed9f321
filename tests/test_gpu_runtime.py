"""Module level: compress -> package -> load -> forward, on the GPU.  Checks the attribute names
the compressor attaches, the safetensors keys / dtypes / rans_info record, and that a model whose
layers were swapped for the compressed modules reproduces the uncompressed model."""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn as nn

pytestmark = pytest.mark.gpu


class Tiny(nn.Module):
    def __init__(self, V=1300, H=128, F=256):
        super().__init__()
        self.embed_tokens = nn.Embedding(V, H)
        self.up_proj = nn.Linear(H, F, bias=True)
        self.down_proj = nn.Linear(F, H, bias=False)
        self.norm = nn.LayerNorm(H)
        self.lm_head = nn.Linear(H, V, bias=False)

    def forward(self, ids):
        h = self.embed_tokens(ids)
        h = h + self.down_proj(torch.nn.functional.silu(self.up_proj(h)))
        return self.lm_head(self.norm(h))


def _forward_fp32_linears(m, ids):
    """Tiny.forward with every linear computed as an fp32 product of the bf16 operands, rounded to bf16 once
    (bias added the way torch adds a bf16 bias to a bf16 output): what the fused operators are measured
    against, torch.matmul on the decompressed weights in fp32."""
    def lin(layer, x):
        y = (x.float() @ layer.weight.float().t()).to(torch.bfloat16)
        return y if layer.bias is None else (y.float() + layer.bias.float()).to(torch.bfloat16)

    h = m.embed_tokens(ids)
    h = h + lin(m.down_proj, torch.nn.functional.silu(lin(m.up_proj, h)))
    return lin(m.lm_head, m.norm(h))


def _make(seed=0):
    torch.manual_seed(seed)
    m = Tiny().to(torch.bfloat16)
    with torch.no_grad():
        for p in m.parameters():
            if p.ndim == 2:
                p.mul_(0.3)
    return m


def test_compress_attributes_and_roundtrip():
    from comp_inference_amd import rans_compress_module_weight, rans_decompress_module_weight

    lin = nn.Linear(256, 128, bias=False).to(torch.bfloat16)
    w = lin.weight.detach().clone()
    rans_compress_module_weight(lin, tile_height=128, tile_width=32)
    assert not hasattr(lin, "weight") and lin.compressed == "rans_bfloat16"
    assert lin.input_shape == [256, 128] and lin.expanded_size == 256 * 128
    for attr in ("exponent_compressed_weight", "exponent_states", "exponent_output_sizes", "exponent_tables",
                 "exponent_slot_map", "exponent_tile_offsets", "exponent_tile_max_lens", "mantissa_raw",
                 "exponent_freqs", "exponent_cdf"):
        assert hasattr(lin, attr), attr
    assert (lin.exponent_num_tiles_k, lin.exponent_num_tiles_n) == (2, 4)
    assert lin.exponent_states.dtype == torch.uint32 and lin.exponent_slot_map.dtype == torch.uint8
    rans_decompress_module_weight(lin)
    assert isinstance(lin.weight, nn.Parameter)
    assert torch.equal(lin.weight.detach().cpu().view(torch.int16), w.t().contiguous().view(torch.int16))
    with pytest.raises(ValueError):
        rans_compress_module_weight(nn.Linear(64, 64, bias=False).to(torch.bfloat16), tile_height=1024)


def test_package_roundtrip_and_forward(tmp_path):
    import comp_inference_amd as ci
    from safetensors import safe_open

    ref = _make()
    ids = torch.tensor([[0, 5, 1299, 640, 5]])
    want = _forward_fp32_linears(ref.cuda(), ids.cuda()).float().cpu()
    ref = ref.cpu()

    comp = _make()
    ci.rans_compress_module_weight(comp.embed_tokens, tile_height=256, tile_width=32, transpose_weight=False)
    ci.rans_compress_module_weight(comp.lm_head, tile_height=256, tile_width=32, transpose_weight=False)
    for name in ("up_proj", "down_proj"):
        ci.rans_compress_module_weight(getattr(comp, name), tile_height=64, tile_width=32)
    out_dir = ci.save_rans_model_package(comp, None, str(tmp_path / "pkg"))
    assert out_dir.endswith("_unfused")
    cfg = json.load(open(os.path.join(out_dir, "config.json")))["quantization_config"]
    assert cfg["quant_method"] == "rans" and cfg["compression"] == "rans_bfloat16"
    assert cfg["layer_configs"]["up_proj"] == {"tile_height": 64, "tile_width": 32, "uncoalesced_interleaving": False}
    path = os.path.join(out_dir, "model.safetensors")
    with safe_open(path, "pt") as f:
        keys = set(f.keys())
        assert f.metadata() == {"format": "pt", "compression_method": "rans_bfloat16", "fused_projections": "False"}
        for mod in ("embed_tokens", "up_proj", "down_proj", "lm_head"):
            for suffix, dt in (("rans_exp_stream", torch.uint8), ("rans_exp_states", torch.uint32),
                               ("rans_exp_tables", torch.uint32), ("rans_exp_slot_map", torch.uint8),
                               ("rans_exp_tile_offsets", torch.uint32), ("rans_exp_tile_max_lens", torch.uint32),
                               ("rans_man_raw", torch.uint8), ("rans_info", torch.int32)):
                assert f"{mod}.{suffix}" in keys
                assert f.get_tensor(f"{mod}.{suffix}").dtype == dt
        assert "up_proj.bias" in keys and "norm.weight" in keys and "up_proj.weight" not in keys
        info = ci.parse_rans_info(f.get_tensor("up_proj.rans_info"))
        assert info["version"] == 1 and info["shape"] == [128, 256] and info["numel"] == 128 * 256
        assert (info["tile_height"], info["tile_width"], info["num_tiles_k"], info["num_tiles_n"]) == (64, 32, 2, 8)

    fresh = _make(seed=123)  # different weights: everything must come from the package
    model = ci.load_compressed_model_with_auto_model("unused", path, model=fresh)
    assert isinstance(model.up_proj, ci.RansLinear) and isinstance(model.embed_tokens, ci.RansEmbedding)
    assert isinstance(model.lm_head, ci.RansLMHead) and model.up_proj.tile_k == 64
    got = model(ids.cuda()).float().cpu()
    assert torch.allclose(got, want, atol=1e-2, rtol=1e-2), (got - want).abs().max()


def test_modules_from_compressed():
    import comp_inference_amd as ci

    torch.manual_seed(1)
    lin = nn.Linear(512, 96, bias=True).to(torch.bfloat16)
    x = torch.randn(3, 512).to(torch.bfloat16)
    want = x.float() @ lin.weight.detach().float().t() + lin.bias.detach().float()  # fp32, decompressed weights
    bias = lin.bias.detach().clone()
    ci.rans_compress_module_weight(lin, tile_height=256, tile_width=32)
    rl = ci.RansLinear.from_compressed(lin, bias=bias)
    got = rl(x.cuda()).float().cpu()
    assert torch.allclose(got, want, atol=1e-2, rtol=1e-2), (got - want).abs().max()
    emb = nn.Embedding(700, 64).to(torch.bfloat16)
    table = emb.weight.detach().clone()
    ci.rans_compress_module_weight(emb, tile_height=256, tile_width=32, transpose_weight=False)
    re = ci.RansEmbedding.from_compressed(emb)
    ids = torch.tensor([0, 699, 300, 300])
    assert torch.equal(re(ids.cuda()).cpu().view(torch.int16), table[ids].view(torch.int16))
    head = ci.RansLMHead(64, 700)
    head.tie_to(re)
    h = torch.randn(2, 64).to(torch.bfloat16)
    assert torch.allclose(head(h.cuda()).float().cpu(), h.float() @ table.float().t(), atol=1e-2, rtol=1e-2)


def test_load_compressed_model_into_skeleton(tmp_path):
    """Package written from compressed modules -> attributes restored on a fresh skeleton ->
    decompressed weights bit-equal to the originals; uncompressed parameters come back as they were."""
    import comp_inference_amd as ci

    src = _make()
    originals = {n: p.detach().clone() for n, p in src.named_parameters()}
    ci.rans_compress_module_weight(src.embed_tokens, tile_height=256, tile_width=32, transpose_weight=False)
    ci.rans_compress_module_weight(src.up_proj, tile_height=64, tile_width=32)
    ci.rans_compress_module_weight(src.down_proj, tile_height=64, tile_width=32, uncoalesced_interleaving=True)
    path = str(tmp_path / "m.safetensors")
    ci.pack_and_save_tensors(src, path)

    dst = _make()
    with torch.no_grad():
        for p in dst.parameters():
            p.add_(1.0)  # make sure nothing of the skeleton's own values survives
    ci.load_compressed_model(dst, path)
    for name in ("embed_tokens", "up_proj", "down_proj"):
        mod = getattr(dst, name)
        assert mod.compressed == "rans_bfloat16" and not hasattr(mod, "weight")
    assert dst.down_proj.exponent_uncoalesced_interleaving and not dst.up_proj.exponent_uncoalesced_interleaving
    assert torch.equal(dst.lm_head.weight.detach(), originals["lm_head.weight"])
    ci.rans_decompress_module_weight(dst.up_proj)
    ci.rans_decompress_module_weight(dst.down_proj)
    ci.rans_decompress_module_weight(dst.embed_tokens)
    assert torch.equal(dst.up_proj.weight.detach().cpu().view(torch.int16),
                       originals["up_proj.weight"].t().contiguous().view(torch.int16))
    assert torch.equal(dst.down_proj.weight.detach().cpu().view(torch.int16),
                       originals["down_proj.weight"].t().contiguous().view(torch.int16))
    assert torch.equal(dst.embed_tokens.weight.detach().cpu().view(torch.int16),
                       originals["embed_tokens.weight"].view(torch.int16))


def _fused_forward(proj, x):
    import comp_inference_amd as ci

    K, N = proj.input_shape
    return ci.fused_rans_linear_triton(
        x=x, compressed_data=proj.exponent_compressed_weight.cuda(), initial_states=proj.exponent_states.cuda(),
        tables=proj.exponent_tables.cuda(), slot_map=proj.exponent_slot_map.cuda(), weight_shape=(K, N),
        tile_offsets=proj.exponent_tile_offsets.cuda(), tile_max_lens=proj.exponent_tile_max_lens.cuda(),
        tile_k=proj.exponent_tile_height, tile_n=proj.exponent_tile_width, mantissas=proj.mantissa_raw.cuda())


def test_fused_qkv_and_gate_up_compression():
    """comp_inference/comp_inference.py:242-341: q/k/v (and gate/up) concatenated along the outputs and
    compressed as one weight under the first projection's name; the reference's own check feeds real
    activations through the fused QKV and compares with torch.matmul (tests/test_fused_model.py:66-95,
    8 rows, K = 1024, N = 4096, max difference below 0.1)."""
    import comp_inference_amd as ci

    torch.manual_seed(3)
    K, Nq, Nkv, F = 1024, 2048, 1024, 3072

    class Attn(nn.Module):
        def __init__(self):
            super().__init__()
            self.q_proj, self.k_proj, self.v_proj = (nn.Linear(K, Nq, bias=False), nn.Linear(K, Nkv, bias=False),
                                                     nn.Linear(K, Nkv, bias=False))

    class Mlp(nn.Module):
        def __init__(self):
            super().__init__()
            self.gate_proj, self.up_proj = nn.Linear(K, F, bias=False), nn.Linear(K, F, bias=False)

    attn, mlp = Attn().to(torch.bfloat16), Mlp().to(torch.bfloat16)
    x = torch.randn(8, K).to(torch.bfloat16).cuda()
    qkv_w = torch.cat([attn.q_proj.weight, attn.k_proj.weight, attn.v_proj.weight], 0).detach().clone()
    gu_w = torch.cat([mlp.gate_proj.weight, mlp.up_proj.weight], 0).detach().clone()

    ci.rans_compress_qkv_fused(attn)
    assert attn.qkv_fused and not hasattr(attn, "k_proj") and not hasattr(attn, "v_proj")
    assert attn.q_proj.input_shape == [K, Nq + 2 * Nkv] and attn.q_proj.compressed == "rans_bfloat16"
    got = _fused_forward(attn.q_proj, x)
    want = torch.matmul(x, qkv_w.cuda().t())
    assert got.shape == (8, Nq + 2 * Nkv) and float((got.float() - want.float()).abs().max()) < 0.1
    assert torch.allclose(got.float(), want.float(), atol=1e-2, rtol=1e-2)
    ci.rans_decompress_module_weight(attn.q_proj)
    assert torch.equal(attn.q_proj.weight.detach().cpu().view(torch.int16), qkv_w.t().contiguous().view(torch.int16))

    ci.rans_compress_gate_up_fused(mlp, tile_height=512, tile_width=32)
    assert mlp.gate_up_fused and not hasattr(mlp, "up_proj")
    assert mlp.gate_proj.input_shape == [K, 2 * F] and mlp.gate_proj.exponent_tile_height == 512
    got = _fused_forward(mlp.gate_proj, x)
    want = torch.matmul(x, gu_w.cuda().t())
    assert torch.allclose(got.float(), want.float(), atol=1e-2, rtol=1e-2)
    ci.rans_decompress_module_weight(mlp.gate_proj)
    assert torch.equal(mlp.gate_proj.weight.detach().cpu().view(torch.int16), gu_w.t().contiguous().view(torch.int16))


def test_rans_linear_prepares_once_and_follows_its_buffers():
    """RansLinear converts its buffers once per device and then reuses the pointers: repeated calls, calls
    with other row counts (also above the decode-once threshold), a module moved to the device, a replaced
    bias and a changed segment count all give what the entry point gives on the same arguments."""
    import comp_inference_amd as ci

    torch.manual_seed(11)
    K, N = 2048, 160
    lin = nn.Linear(K, N, bias=True).to(torch.bfloat16)
    bias = lin.bias.detach().clone()
    ci.rans_compress_module_weight(lin)
    rl = ci.RansLinear.from_compressed(lin, bias=bias)

    def entry(x, b, segments):
        ck = None
        if segments > 1:
            ck = ci.build_checkpoints(rl.rans_exp_stream.cuda(), rl.rans_exp_states.cuda(), rl.rans_exp_tables.cuda(),
                                      rl.rans_exp_slot_map.cuda(), (K, N), rl.rans_exp_tile_offsets.cuda(),
                                      rl.rans_exp_tile_max_lens.cuda(), rl.tile_k, rl.tile_n, segments)
        return ci.fused_rans_linear_triton(
            x=x, compressed_data=rl.rans_exp_stream.cuda(), initial_states=rl.rans_exp_states.cuda(),
            tables=rl.rans_exp_tables.cuda(), slot_map=rl.rans_exp_slot_map.cuda(), weight_shape=(K, N),
            tile_offsets=rl.rans_exp_tile_offsets.cuda(), tile_max_lens=rl.rans_exp_tile_max_lens.cuda(),
            tile_k=rl.tile_k, tile_n=rl.tile_n, mantissas=rl.rans_man_raw.cuda(), bias=b.cuda(),
            checkpoints=ck, segments=segments)

    def same(a, b):
        return torch.equal(a.view(torch.int16), b.view(torch.int16))

    segs = rl._checkpoints(torch.device("cuda", 0))[1]
    xs = {M: torch.randn(M, K).to(torch.bfloat16).cuda() for M in (1, 5, 64, 70)}
    for M in (1, 5, 1, 64, 70, 5):                       # buffers on the host: device copies are kept
        assert same(rl(xs[M]), entry(xs[M], bias, segs)), M
    first = rl._prepared[1]
    assert rl(xs[1][None]).shape == (1, 1, N) and rl._prepared[1] is first

    rl = rl.cuda()                                       # the buffers are new tensors now
    assert same(rl(xs[5]), entry(xs[5], bias, segs)) and rl._prepared[1] is not first
    assert rl._prepared[1].keep[0].data_ptr() == rl.rans_exp_stream.data_ptr()      # no second copy

    rl.bias = (bias.float() + 1).to(torch.bfloat16).cuda()
    assert same(rl(xs[5]), entry(xs[5], rl.bias, segs))
    rl.segments = 1 if segs > 1 else 2
    assert same(rl(xs[5]), entry(xs[5], rl.bias, rl.segments))
    with pytest.raises(RuntimeError):
        rl(xs[5].cpu())
    with pytest.raises(RuntimeError):
        rl._prepared[1](xs[5].cpu())

    import copy                                          # a copy of the module points at its own tensors
    want = rl(xs[5])
    twin = copy.deepcopy(rl)
    call = twin._prepared[1]
    assert call is not rl._prepared[1] and call.keep[0] is twin.rans_exp_stream
    assert call.keep[0].data_ptr() != rl.rans_exp_stream.data_ptr()
    assert call.p[0].value == call.keep[0].data_ptr() and call.p[6].value == call.keep[6].data_ptr()
    del rl
    assert same(twin(xs[5]), want)


def test_gguf_export_holds_the_weights(tmp_path):
    """comp_inference/rans_gguf.py:111-238 stores states, sizes, freqs and cdf but neither tables nor tile
    offsets: all of them follow from what is stored (tables = freq | cdf << 16, a tile's length = its longest
    stream, offsets = running sum).  Rebuilt that way from the file alone, every weight decodes to its
    original bits."""
    import types

    from gguf_parse import parse_gguf

    import comp_inference_amd as ci
    from comp_inference_amd.rans_gguf import save_rans_model_gguf

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.mlp = nn.Module()
            self.mlp.up_proj = nn.Linear(1100, 200, bias=True)
            self.mlp.down_proj = nn.Linear(200, 1100, bias=False)

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.model = nn.Module()
            self.model.embed_tokens = nn.Embedding(1300, 96)
            self.model.layers = nn.ModuleList([Block()])
            self.config = types.SimpleNamespace(num_hidden_layers=1, hidden_size=96, intermediate_size=200,
                                                num_attention_heads=4)

    torch.manual_seed(21)
    net = Net().to(torch.bfloat16)
    up, down, emb = net.model.layers[0].mlp.up_proj, net.model.layers[0].mlp.down_proj, net.model.embed_tokens
    want = {"blk.0.ffn_up": up.weight.detach().t().contiguous(), "blk.0.ffn_down": down.weight.detach().t().contiguous(),
            "token_embd": emb.weight.detach().clone()}
    ci.rans_compress_module_weight(up)
    ci.rans_compress_module_weight(down, tile_height=64, tile_width=32)
    ci.rans_compress_module_weight(emb, transpose_weight=False)
    tiles = {"blk.0.ffn_up": (1024, 32), "blk.0.ffn_down": (64, 32), "token_embd": (1024, 32)}

    class Tok:
        bos_token_id = eos_token_id = pad_token_id = None
        all_special_ids = []
        backend_tokenizer = types.SimpleNamespace(model=types.SimpleNamespace(get_merges=lambda: ["a b"]))

        def get_vocab(self):
            return {"a": 0, "b": 1, "ab": 2}

    path = tmp_path / "net.gguf"
    save_rans_model_gguf(net, Tok(), str(path))
    _, _, tensors, _, _ = parse_gguf(path)

    def u(name, dtype):
        return torch.from_numpy(tensors[name][0].copy()).view(dtype)

    for base, w in want.items():
        info = tensors[f"{base}.rans_info"][0].tolist()
        K, N = info[7:9]
        th, tw = tiles[base]
        assert info[:7] == [1, K * N, 1, -(-K // th) * -(-N // tw) * 2 * tw, 0, 0, 2] and (K, N) == tuple(w.shape)
        freqs, cdf = u(f"{base}.rans_exp_freqs", torch.uint16), u(f"{base}.rans_exp_cdf", torch.uint16)
        f64, c64 = freqs.to(torch.int64), cdf.to(torch.int64)
        tables = (f64 | (c64 << 16)).to(torch.uint32)
        slot_map = torch.repeat_interleave(torch.arange(256), f64).to(torch.uint8)
        assert slot_map.numel() == 4096
        sizes = u(f"{base}.rans_exp_sizes", torch.uint32).to(torch.int64).view(-1, 2 * tw)
        max_lens = sizes.max(dim=1).values
        offsets = torch.cumsum(max_lens * 2 * tw, 0) - max_lens * 2 * tw
        stream = u(f"{base}.rans_exp_stream", torch.uint8)
        assert stream.numel() == int((max_lens * 2 * tw).sum())
        exp = ci.rans_decomp_triton_tiled(stream.cuda(), u(f"{base}.rans_exp_states", torch.uint32).cuda(),
                                          tables.cuda(), slot_map.cuda(), (K, N), offsets.to(torch.uint32).cuda(),
                                          max_lens.to(torch.uint32).cuda(), tile_k=th, tile_n=tw)
        man = ci.uninterleave_mantissas(u(f"{base}.rans_man_raw", torch.uint8), K, N, TILE_K=th, TILE_N=tw)
        got = ci.reconstruct_from_exp_and_mantissa(exp.cpu(), man)
        assert torch.equal(got.view(torch.int16), w.view(torch.int16)), base
    assert torch.equal(u("blk.0.ffn_up.bias", torch.float32), up.bias.detach().float())


def test_tied_head_package_ties_the_head_to_the_compressed_table(tmp_path):
    """A model whose head shares the embedding table, saved with tied_lm_head=True: the file holds the compressed
    table once and no lm_head.weight (comp_inference/rans_saving.py:186-191); loaded into a freshly built model
    (nothing pretrained behind it) the head must be tied to the compressed table, not left at its random
    initialisation.  With the head compressed as well its tensors stay in the file, as in the reference."""
    import comp_inference_amd as ci
    from safetensors import safe_open

    class TinyTied(Tiny):
        def get_input_embeddings(self):
            return self.embed_tokens

    def make(seed):
        torch.manual_seed(seed)
        m = TinyTied().to(torch.bfloat16)
        with torch.no_grad():
            for p in m.parameters():
                if p.ndim == 2:
                    p.mul_(0.3)
        m.lm_head.weight = m.embed_tokens.weight
        return m

    ref = make(0)
    ids = torch.tensor([[3, 17, 1299, 640]])
    want = _forward_fp32_linears(ref.cuda(), ids.cuda()).float().cpu()
    comp = make(0)
    ci.rans_compress_module_weight(comp.embed_tokens, tile_height=256, tile_width=32, transpose_weight=False)
    for name in ("up_proj", "down_proj"):
        ci.rans_compress_module_weight(getattr(comp, name), tile_height=64, tile_width=32)
    out_dir = ci.save_rans_model_package(comp, None, str(tmp_path / "tied"), tied_lm_head=True)
    path = os.path.join(out_dir, "model.safetensors")
    with safe_open(path, "pt") as f:
        keys = set(f.keys())
    assert "embed_tokens.rans_exp_stream" in keys and "lm_head.weight" not in keys and "lm_head.rans_exp_stream" not in keys
    model = ci.load_compressed_model_with_auto_model("unused", path, model=make(77))
    assert isinstance(model.lm_head, ci.RansLMHead) and isinstance(model.embed_tokens, ci.RansEmbedding)
    assert model.lm_head.rans_exp_stream.data_ptr() == model.embed_tokens.rans_exp_stream.data_ptr()  # on the GPU once
    got = model(ids.cuda()).float().cpu()
    assert torch.allclose(got, want, atol=1e-2, rtol=1e-2), (got - want).abs().max()

    # head compressed too: its tensors are written although the head is tied
    both = make(0)
    both.lm_head.weight = nn.Parameter(both.embed_tokens.weight.detach().clone())
    ci.rans_compress_module_weight(both.embed_tokens, tile_height=256, tile_width=32, transpose_weight=False)
    ci.rans_compress_module_weight(both.lm_head, tile_height=256, tile_width=32, transpose_weight=False)
    tensors = ci.rans_saving.collect_tensors(both, tied_lm_head=True)
    assert "lm_head.rans_exp_stream" in tensors and "lm_head.weight" not in tensors


def test_transformers_model_from_its_package_directory(tmp_path):
    """The loader's own path (comp_inference/pytorch_runtime.py:552-642 with a local directory for model_id): the
    package written from a transformers model holds config.json with the quantization block; the model is built
    from that config alone, every compressed module is swapped in with the tile shape its layer_configs entry
    names (none of them the default here), and the logits are those of the model on its decompressed weights."""
    transformers = pytest.importorskip("transformers")
    import comp_inference_amd as ci

    cfg = transformers.LlamaConfig(vocab_size=300, hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                                   num_attention_heads=2, num_key_value_heads=1, max_position_embeddings=64,
                                   tie_word_embeddings=False)
    torch.manual_seed(0)
    ref = transformers.LlamaForCausalLM(cfg).to(torch.bfloat16).eval()
    ids = torch.tensor([[1, 17, 299, 64, 5]])
    with torch.no_grad():
        want = ref(ids).logits.float()
    comp = transformers.LlamaForCausalLM(cfg).to(torch.bfloat16).eval()
    comp.load_state_dict(ref.state_dict())
    for name, mod in list(comp.named_modules()):
        if isinstance(mod, nn.Embedding) or name == "lm_head":
            ci.rans_compress_module_weight(mod, tile_height=128, tile_width=32, transpose_weight=False)
        elif isinstance(mod, nn.Linear):
            ci.rans_compress_module_weight(mod, tile_height=64, tile_width=32)
    out_dir = ci.save_rans_model_package(comp, None, str(tmp_path / "llama"))
    saved = json.load(open(os.path.join(out_dir, "config.json")))
    assert saved["model_type"] == "llama" and saved["quantization_config"]["quant_method"] == "rans"
    assert saved["quantization_config"]["layer_configs"]["model.layers.1.mlp.down_proj"]["tile_height"] == 64

    model = ci.load_compressed_model_with_auto_model(out_dir, os.path.join(out_dir, "model.safetensors"))
    assert isinstance(model.model.embed_tokens, ci.RansEmbedding) and model.model.embed_tokens.tile_k == 128
    assert isinstance(model.lm_head, ci.RansLMHead) and model.lm_head.tile_k == 128
    layer = model.model.layers[1]
    for lin in (layer.self_attn.q_proj, layer.self_attn.k_proj, layer.self_attn.o_proj, layer.mlp.gate_proj, layer.mlp.down_proj):
        assert isinstance(lin, ci.RansLinear) and lin.tile_k == 64
    assert torch.equal(model.model.norm.weight.detach().cpu(), ref.model.norm.weight.detach())
    with torch.no_grad():
        got = model(ids.cuda()).logits.float().cpu()
    # (bf16 activations between the layers: a different summation order moves a logit by a bf16 step or two)
    assert torch.allclose(got, want, atol=5e-2, rtol=5e-2), (got - want).abs().max()
    assert (got.argmax(-1) == want.argmax(-1)).float().mean() >= 0.8


def test_reloading_buffers_in_place_is_noticed():
    """The loader's idiom replaces `tensor.data` under the same tensor objects: a module that has already run
    must drop what it prepared from the old storage (pointers, checkpoints, slot table) and use the new weight."""
    import comp_inference_amd as ci

    def compressed(seed):
        torch.manual_seed(seed)
        lin = nn.Linear(2048, 64, bias=False).to(torch.bfloat16)
        w = lin.weight.detach().clone()
        ci.rans_compress_module_weight(lin, tile_height=1024, tile_width=32)
        return ci.RansLinear.from_compressed(lin).cuda(), w

    a, wa = compressed(1)
    b, wb = compressed(2)
    x = torch.randn(2, 2048).to(torch.bfloat16).cuda()
    ya = a(x).float().cpu()
    assert torch.allclose(ya, x.float().cpu() @ wa.float().t(), atol=1e-2, rtol=1e-2)
    for name, buf in a.named_buffers():
        buf.data = dict(b.named_buffers())[name].data.clone()
    yb = a(x).float().cpu()
    assert torch.allclose(yb, x.float().cpu() @ wb.float().t(), atol=1e-2, rtol=1e-2)
    assert torch.equal(yb, b(x).float().cpu())
    assert ci.release_scratch() >= 0


def test_rans_linear_that_keeps_nothing_on_the_device():
    """RansLinear.resident = False: the reference's forward (comp_inference/pytorch_runtime.py:440-459) -- the
    buffers stay where they are (here: on the host), every call moves them to the input's device and drops the
    copies; the result is the entry point's on the same arguments, and nothing is kept on the module."""
    import comp_inference_amd as ci

    torch.manual_seed(5)
    K, N = 1024, 96
    lin = nn.Linear(K, N, bias=True).to(torch.bfloat16)
    w, bias = lin.weight.detach().clone(), lin.bias.detach().clone()
    ci.rans_compress_module_weight(lin, tile_height=512, tile_width=32)
    rl = ci.RansLinear.from_compressed(lin, bias=bias)
    rl.resident = False
    for M in (1, 3, 70):
        x = torch.randn(M, K).to(torch.bfloat16).cuda()
        got = rl(x)
        want = ci.fused_rans_linear_triton(
            x=x, compressed_data=rl.rans_exp_stream.cuda(), initial_states=rl.rans_exp_states.cuda(),
            tables=rl.rans_exp_tables.cuda(), slot_map=rl.rans_exp_slot_map.cuda(), weight_shape=(K, N),
            tile_offsets=rl.rans_exp_tile_offsets.cuda(), tile_max_lens=rl.rans_exp_tile_max_lens.cuda(),
            tile_k=rl.tile_k, tile_n=rl.tile_n, mantissas=rl.rans_man_raw.cuda(), bias=bias.cuda())
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
        ref = x.float().cpu() @ w.float().t() + bias.float()
        assert torch.allclose(got.float().cpu(), ref, atol=1e-2, rtol=1e-2)
    assert not hasattr(rl, "_prepared") and not hasattr(rl, "_ckpt_cache")
    assert rl.rans_exp_stream.device.type == "cpu"
    rl.resident = True  # back to the prepared call: a device copy and the checkpoint index are kept from here on
    assert torch.allclose(rl(x).float().cpu(), ref, atol=1e-2, rtol=1e-2) and hasattr(rl, "_prepared")
