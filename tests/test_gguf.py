"""GGUF export (comp_inference/rans_gguf.py:111-238): container layout, metadata keys and order, tensor
names / dtypes / contents.  The reference writes through the third-party `gguf` package, which is absent
here and has no test reading a file back, so the check is against the published GGUF v3 layout, read by
an independent parser (tests/gguf_parse.py).  No GPU: modules carry synthetic compressed attributes."""
import json
import types

import numpy as np
import pytest
import torch
import torch.nn as nn

from gguf_parse import parse_gguf


class _Tok:
    bos_token_id, eos_token_id, pad_token_id = 1, 2, None
    all_special_ids = [1, 2, 99]

    def get_vocab(self):
        return {"<s>": 1, "</s>": 2, "a": 0, "b": 3, "ab": 4, "": 5, "é": 6}     # empty token -> <unk>


def _tokenizer_dir(tmp_path, merges):
    (tmp_path / "tokenizer.json").write_text(json.dumps({"model": {"merges": merges}}))
    return str(tmp_path)


class _Layer(nn.Module):
    def __init__(self, H, F):
        super().__init__()
        self.self_attn = nn.Module()
        self.self_attn.q_proj = nn.Linear(H, H, bias=True)
        self.self_attn.o_proj = nn.Linear(H, H, bias=False)
        self.mlp = nn.Module()
        self.mlp.down_proj = nn.Linear(F, H, bias=False)
        self.input_layernorm = nn.LayerNorm(H, bias=False)
        self.post_attention_layernorm = nn.LayerNorm(H, bias=False)


class _Model(nn.Module):
    def __init__(self, H=8, F=16, V=7):
        super().__init__()
        self.model = nn.Module()
        self.model.embed_tokens = nn.Embedding(V, H)
        self.model.layers = nn.ModuleList([_Layer(H, F), _Layer(H, F)])
        self.model.norm = nn.LayerNorm(H, bias=False)
        self.lm_head = nn.Linear(H, V, bias=False)
        self.config = types.SimpleNamespace(num_hidden_layers=2, hidden_size=H, intermediate_size=F,
                                            num_attention_heads=2, num_key_value_heads=1, rope_theta=5e5,
                                            rms_norm_eps=1e-5)


def _fake_compress(mod, seed, raw_exponent=False):
    """The attributes `rans_compress_module_weight` leaves (comp_inference/comp_inference.py:368-487),
    filled with arbitrary bytes: the export only moves them."""
    g = torch.Generator().manual_seed(seed)
    K, N = mod.weight.shape[1], mod.weight.shape[0]
    mod.input_shape, mod.expanded_size, mod.compressed = [K, N], K * N, "rans_bfloat16"
    if raw_exponent:
        mod.exponent_raw = torch.randint(0, 256, (K, N), generator=g).to(torch.uint8)
    else:
        mod.exponent_compressed_weight = torch.randint(0, 256, (37 + seed,), generator=g).to(torch.uint8)
        mod.exponent_states = torch.randint(1 << 16, 1 << 24, (64,), generator=g).to(torch.uint32)
        mod.exponent_output_sizes = torch.randint(0, 9, (64,), generator=g).to(torch.uint32)
        mod.exponent_freqs = torch.randint(1, 4096, (256,), generator=g).to(torch.uint16)
        mod.exponent_cdf = torch.randint(0, 4096, (256,), generator=g).to(torch.uint16)
        mod.exponent_num_streams = 64
    mod.mantissa_raw = torch.randint(0, 256, (1, 1024, 32), generator=g).to(torch.uint8)
    del mod.weight


def test_name_mapping():
    from comp_inference_amd.rans_gguf import hf_to_gguf_name

    assert hf_to_gguf_name("model.layers.17.self_attn.q_proj") == "blk.17.attn_q"
    assert hf_to_gguf_name("model.layers.0.self_attn.k_proj.weight") == "blk.0.attn_k"
    assert hf_to_gguf_name("model.layers.3.self_attn.v_proj.bias") == "blk.3.attn_v.bias"
    assert hf_to_gguf_name("model.layers.3.self_attn.o_proj") == "blk.3.attn_output"
    assert hf_to_gguf_name("model.layers.3.mlp.gate_proj") == "blk.3.ffn_gate"
    assert hf_to_gguf_name("model.layers.3.mlp.up_proj") == "blk.3.ffn_up"
    assert hf_to_gguf_name("model.layers.3.mlp.down_proj") == "blk.3.ffn_down"
    assert hf_to_gguf_name("model.layers.3.input_layernorm.weight") == "blk.3.attn_norm"
    assert hf_to_gguf_name("model.layers.3.post_attention_layernorm.weight") == "blk.3.ffn_norm"
    assert hf_to_gguf_name("model.embed_tokens") == "token_embd"
    assert hf_to_gguf_name("model.norm.weight") == "output_norm"
    assert hf_to_gguf_name("lm_head") == "output"
    assert hf_to_gguf_name("x.model.layers.3") == "x.model.layers.3"          # only a leading path is rewritten


def test_export_layout_metadata_and_tensors(tmp_path):
    from comp_inference_amd.rans_gguf import save_rans_model_gguf

    torch.manual_seed(0)
    m = _Model().to(torch.bfloat16)
    m.model.norm.float()                                                       # one fp32 parameter
    want_plain = {"output_norm": m.model.norm.weight.detach().clone(),
                  "blk.1.attn_norm": m.model.layers[1].input_layernorm.weight.detach().clone(),
                  "blk.0.attn_output": m.model.layers[0].self_attn.o_proj.weight.detach().clone()}
    q0 = m.model.layers[0].self_attn.q_proj
    _fake_compress(q0, 1)
    _fake_compress(m.model.layers[1].mlp.down_proj, 2, raw_exponent=True)
    _fake_compress(m.model.embed_tokens, 3)
    m.model.embed_tokens.input_shape = []                                      # flat fallback: [numel]
    out = tmp_path / "m.gguf"
    save_rans_model_gguf(m, _Tok(), str(out), _tokenizer_dir(tmp_path, [["a", "b"], "ab é"]))

    version, kvs, tensors, alignment, data_start = parse_gguf(out)
    assert version == 3 and alignment == 32 and data_start % 32 == 0
    keys = [k for k, _, _ in kvs]
    assert keys == ["general.architecture", "qwen3.block_count", "qwen3.context_length", "qwen3.embedding_length",
                    "qwen3.feed_forward_length", "qwen3.attention.head_count", "qwen3.attention.head_count_kv",
                    "qwen3.rope.dimension_count", "qwen3.rope.freq_base", "qwen3.attention.layer_norm_rms_epsilon",
                    "quantization.method", "tokenizer.ggml.model", "tokenizer.ggml.pre", "tokenizer.ggml.merges",
                    "tokenizer.ggml.tokens", "tokenizer.ggml.token_type", "tokenizer.ggml.scores",
                    "tokenizer.ggml.bos_token_id", "tokenizer.ggml.eos_token_id"]          # no pad id: key absent
    kv = {k: (vt, v) for k, vt, v in kvs}
    assert kv["general.architecture"] == (8, b"qwen3") and kv["quantization.method"] == (8, b"rans_bfloat16")
    assert kv["qwen3.block_count"] == (4, 2) and kv["qwen3.context_length"] == (4, 32768)
    assert kv["qwen3.embedding_length"] == (4, 8) and kv["qwen3.feed_forward_length"] == (4, 16)
    assert kv["qwen3.attention.head_count"] == (4, 2) and kv["qwen3.attention.head_count_kv"] == (4, 1)
    assert kv["qwen3.rope.dimension_count"] == (4, 4)
    assert kv["qwen3.rope.freq_base"] == (6, 5e5)
    assert kv["qwen3.attention.layer_norm_rms_epsilon"] == (6, float(np.float32(1e-5)))
    assert kv["tokenizer.ggml.model"] == (8, b"gpt2") and kv["tokenizer.ggml.pre"] == (8, b"qwen2")
    assert kv["tokenizer.ggml.merges"] == (9, (8, [b"a b", "ab é".encode()]))
    assert kv["tokenizer.ggml.tokens"] == (9, (8, [b"a", b"<s>", b"</s>", b"b", b"ab", b"<unk>", "é".encode()]))
    assert kv["tokenizer.ggml.token_type"] == (9, (5, [1, 3, 3, 1, 1, 1, 1]))
    assert kv["tokenizer.ggml.scores"] == (9, (6, [0.0] * 7))
    assert kv["tokenizer.ggml.bos_token_id"] == (4, 1) and kv["tokenizer.ggml.eos_token_id"] == (4, 2)

    def same(name, t, np_dtype):
        a = tensors[name][0]
        assert a.dtype == np.dtype(np_dtype) and a.shape == tuple(t.shape), name
        assert a.tobytes() == t.detach().contiguous().cpu().view(torch.uint8).numpy().tobytes(), name

    same("blk.0.attn_q.rans_exp_stream", q0.exponent_compressed_weight, np.int8)
    same("blk.0.attn_q.rans_exp_states", q0.exponent_states, np.int32)
    same("blk.0.attn_q.rans_exp_sizes", q0.exponent_output_sizes, np.int32)
    same("blk.0.attn_q.rans_exp_freqs", q0.exponent_freqs, np.int16)
    same("blk.0.attn_q.rans_exp_cdf", q0.exponent_cdf, np.int16)
    same("blk.0.attn_q.rans_man_raw", q0.mantissa_raw.flatten(), np.int8)
    same("blk.0.attn_q.bias", q0.bias.float(), np.float32)
    assert tensors["blk.0.attn_q.rans_info"][0].tolist() == [1, 64, 1, 64, 0, 0, 2, 8, 8]
    dp = m.model.layers[1].mlp.down_proj
    same("blk.1.ffn_down.rans_exp_raw", dp.exponent_raw, np.int8)              # 2-d: dims stored reversed
    assert tensors["blk.1.ffn_down.rans_info"][0].tolist() == [1, 128, 0, 0, 0, 0, 2, 16, 8]
    assert "blk.1.ffn_down.rans_exp_stream" not in tensors and "blk.1.ffn_down.bias" not in tensors
    assert tensors["token_embd.rans_info"][0].tolist() == [1, 56, 1, 64, 0, 0, 1, 56]
    same("output_norm", want_plain["output_norm"], np.float32)
    same("blk.1.attn_norm", want_plain["blk.1.attn_norm"], np.int16)           # bf16 bits
    same("blk.0.attn_output", want_plain["blk.0.attn_output"], np.int16)
    assert "blk.0.attn_q" not in tensors and "blk.0.attn_q.weight" not in tensors
    # directory order = module order; every offset aligned (checked by the parser) and increasing
    offs = [off for _, off in tensors.values()]
    assert offs == sorted(offs) and list(tensors)[0] == "token_embd.rans_exp_stream"


def test_export_needs_merges(tmp_path):
    from comp_inference_amd.rans_gguf import save_rans_model_gguf

    with pytest.raises(ValueError, match="merges"):
        save_rans_model_gguf(_Model(), _Tok(), str(tmp_path / "x.gguf"), str(tmp_path))

    class Backend(_Tok):                                                       # merges from the tokenizer itself
        backend_tokenizer = types.SimpleNamespace(model=types.SimpleNamespace(get_merges=lambda: [("a", "b")]))

    save_rans_model_gguf(_Model(), Backend(), str(tmp_path / "y.gguf"), None)
    _, kvs, tensors, _, _ = parse_gguf(tmp_path / "y.gguf")
    assert dict((k, v) for k, _, v in kvs)["tokenizer.ggml.merges"] == (8, [b"a b"])
    assert tensors["output"][0].shape == (7, 8) and "blk.0.attn_q.bias" in tensors
