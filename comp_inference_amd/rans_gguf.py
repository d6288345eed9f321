"""GGUF export of a compressed model (comp_inference/rans_gguf.py:111-238).

The reference drives the third-party `gguf` package (unpinned in its pyproject, absent here); this
module writes the container itself, following the published GGUF v3 layout:

    header   : magic "GGUF", u32 version = 3, u64 tensor count, u64 key/value count      (little endian)
    metadata : per entry  string key, u32 value type, value
               string = u64 length + UTF-8 bytes; array = u32 element type, u64 count, elements
    tensors  : per tensor string name, u32 rank, u64 dims[rank] (fastest-varying first, i.e. the
               numpy shape reversed), u32 ggml type, u64 offset into the data section
    padding to `general.alignment` (32), then the data section: each tensor padded to the alignment.

Keys, tensor names, dtypes and their order are the reference's: the `add_*` helpers of the package map
to the key names given in `_Writer` below.  Container plumbing only: no arithmetic of the hot path.
"""
from __future__ import annotations

import json
import os
import re
import struct

import numpy as np
import torch

GGUF_MAGIC = 0x46554747          # "GGUF" read as a little-endian u32
GGUF_VERSION = 3
GGUF_ALIGNMENT = 32

# metadata value types
T_UINT8, T_INT8, T_UINT16, T_INT16, T_UINT32, T_INT32, T_FLOAT32, T_BOOL, T_STRING, T_ARRAY, T_UINT64, T_INT64, \
    T_FLOAT64 = range(13)
_SCALAR_FMT = {T_UINT8: "<B", T_INT8: "<b", T_UINT16: "<H", T_INT16: "<h", T_UINT32: "<I", T_INT32: "<i",
               T_FLOAT32: "<f", T_BOOL: "<?", T_UINT64: "<Q", T_INT64: "<q", T_FLOAT64: "<d"}

# ggml tensor types for the numpy dtypes the export produces
GGML_TYPE = {np.dtype(np.float32): 0, np.dtype(np.float16): 1, np.dtype(np.int8): 24, np.dtype(np.int16): 25,
             np.dtype(np.int32): 26, np.dtype(np.int64): 27, np.dtype(np.float64): 28}


def hf_to_gguf_name(name: str) -> str:
    """Hugging Face module path -> llama.cpp tensor name (comp_inference/rans_gguf.py:11-28)."""
    out = re.sub(r"^model\.layers\.(\d+)", r"blk.\1", name)
    for old, new in (("model.embed_tokens", "token_embd"), ("model.norm", "output_norm"), ("lm_head", "output"),
                     ("self_attn.q_proj", "attn_q"), ("self_attn.k_proj", "attn_k"), ("self_attn.v_proj", "attn_v"),
                     ("self_attn.o_proj", "attn_output"), ("mlp.gate_proj", "ffn_gate"), ("mlp.up_proj", "ffn_up"),
                     ("mlp.down_proj", "ffn_down"), ("input_layernorm", "attn_norm"),
                     ("post_attention_layernorm", "ffn_norm")):
        out = out.replace(old, new)
    return out[:-7] if out.endswith(".weight") else out


def sanitize_merges(raw_merges):
    """BPE merges as "left right" strings whichever way the tokenizer stores them
    (comp_inference/rans_gguf.py:30-42)."""
    out = []
    for m in raw_merges or []:
        if isinstance(m, str):
            out.append(m)
        elif hasattr(m, "__getitem__") and len(m) >= 2:
            out.append(f"{m[0]} {m[1]}")
        else:
            out.append(str(m))
    return out


def _string(s) -> bytes:
    b = s if isinstance(s, (bytes, bytearray)) else str(s).encode("utf-8")
    return struct.pack("<Q", len(b)) + bytes(b)


class _Writer:
    """The subset of the package's writer the export uses; each method names the key it writes."""

    def __init__(self, path: str, arch: str):
        self.path, self.arch = path, arch
        self.kv: dict[str, bytes] = {}           # insertion-ordered; a repeated key overrides in place
        self.tensors: list[tuple[str, np.ndarray]] = []

    # ---- metadata
    def _put(self, key: str, vtype: int, payload: bytes) -> None:
        self.kv[key] = struct.pack("<I", vtype) + payload

    def add_string(self, key, val):
        self._put(key, T_STRING, _string(val))

    def add_uint32(self, key, val):
        self._put(key, T_UINT32, struct.pack("<I", int(val)))

    def add_float32(self, key, val):
        self._put(key, T_FLOAT32, struct.pack("<f", float(val)))

    def add_array(self, key, values):
        """Element type from the first element, as the package does: bytes/str -> string, float -> f32,
        bool -> bool, int -> i32."""
        values = list(values)
        if not values:
            raise ValueError(f"empty array for {key!r}")
        first = values[0]
        if isinstance(first, (str, bytes, bytearray)):
            et, body = T_STRING, b"".join(_string(v) for v in values)
        elif isinstance(first, bool):
            et, body = T_BOOL, np.asarray(values, dtype=np.bool_).tobytes()
        elif isinstance(first, float):
            et, body = T_FLOAT32, np.asarray(values, dtype="<f4").tobytes()
        elif isinstance(first, (int, np.integer)):
            et, body = T_INT32, np.asarray(values, dtype="<i4").tobytes()
        else:
            raise ValueError(f"unsupported array element {type(first).__name__} for {key!r}")
        self._put(key, T_ARRAY, struct.pack("<IQ", et, len(values)) + body)

    def add_architecture(self):
        self.add_string("general.architecture", self.arch)

    def add_block_count(self, n):
        self.add_uint32(f"{self.arch}.block_count", n)

    def add_context_length(self, n):
        self.add_uint32(f"{self.arch}.context_length", n)

    def add_embedding_length(self, n):
        self.add_uint32(f"{self.arch}.embedding_length", n)

    def add_feed_forward_length(self, n):
        self.add_uint32(f"{self.arch}.feed_forward_length", n)

    def add_head_count(self, n):
        self.add_uint32(f"{self.arch}.attention.head_count", n)

    def add_head_count_kv(self, n):
        self.add_uint32(f"{self.arch}.attention.head_count_kv", n)

    def add_rope_dimension_count(self, n):
        self.add_uint32(f"{self.arch}.rope.dimension_count", n)

    def add_rope_freq_base(self, v):
        self.add_float32(f"{self.arch}.rope.freq_base", v)

    def add_layer_norm_rms_eps(self, v):
        self.add_float32(f"{self.arch}.attention.layer_norm_rms_epsilon", v)

    def add_tokenizer_model(self, s):
        self.add_string("tokenizer.ggml.model", s)

    def add_tokenizer_pre(self, s):
        self.add_string("tokenizer.ggml.pre", s)

    def add_token_merges(self, merges):
        self.add_array("tokenizer.ggml.merges", merges)

    def add_token_list(self, tokens):
        self.add_array("tokenizer.ggml.tokens", tokens)

    def add_token_types(self, types):
        self.add_array("tokenizer.ggml.token_type", types)

    def add_token_scores(self, scores):
        self.add_array("tokenizer.ggml.scores", scores)

    def add_bos_token_id(self, i):
        self.add_uint32("tokenizer.ggml.bos_token_id", i)

    def add_eos_token_id(self, i):
        self.add_uint32("tokenizer.ggml.eos_token_id", i)

    def add_pad_token_id(self, i):
        self.add_uint32("tokenizer.ggml.padding_token_id", i)

    # ---- tensors
    def add_tensor(self, name: str, data: np.ndarray) -> None:
        if data.dtype not in GGML_TYPE:
            raise ValueError(f"tensor {name!r}: dtype {data.dtype} has no ggml type")
        if any(name == n for n, _ in self.tensors):
            raise ValueError(f"duplicated tensor name {name!r}")
        self.tensors.append((name, np.ascontiguousarray(data)))

    def write(self) -> None:
        def pad(n):
            return (-n) % GGUF_ALIGNMENT

        infos, offset = [], 0
        for name, a in self.tensors:
            dims = a.shape[::-1] if a.ndim else (1,)
            infos.append(_string(name) + struct.pack("<I", len(dims)) + struct.pack(f"<{len(dims)}Q", *dims)
                         + struct.pack("<IQ", GGML_TYPE[a.dtype], offset))
            offset += a.nbytes + pad(a.nbytes)
        with open(self.path, "wb") as f:
            f.write(struct.pack("<IIQQ", GGUF_MAGIC, GGUF_VERSION, len(self.tensors), len(self.kv)))
            for key, payload in self.kv.items():
                f.write(_string(key) + payload)
            for info in infos:
                f.write(info)
            f.write(b"\0" * pad(f.tell()))
            for _, a in self.tensors:
                a.astype(a.dtype.newbyteorder("<"), copy=False).tofile(f)
                f.write(b"\0" * pad(a.nbytes))


def write_tokenizer(writer: _Writer, tokenizer, model_path_or_name) -> None:
    """GPT-2 style BPE vocabulary and merges (comp_inference/rans_gguf.py:45-109).  The merges come from
    the tokenizer's backend, else from `tokenizer.json` under `model_path_or_name` (a local directory;
    the reference also asks the hub cache, which is tried only if `transformers` finds the file offline)."""
    merges = []
    if hasattr(tokenizer, "backend_tokenizer"):
        try:
            merges = sanitize_merges(tokenizer.backend_tokenizer.model.get_merges())
        except Exception:
            merges = []
    if not merges and model_path_or_name is not None:
        json_path = os.path.join(str(model_path_or_name), "tokenizer.json")
        if not os.path.exists(json_path):
            try:
                from transformers.utils.hub import cached_file

                json_path = cached_file(model_path_or_name, "tokenizer.json", local_files_only=True)
            except Exception:
                json_path = None
        if json_path and os.path.exists(json_path):
            try:
                with open(json_path, "r", encoding="utf-8") as f:
                    merges = sanitize_merges(json.load(f).get("model", {}).get("merges", []))
            except Exception:
                merges = []
    if not merges:
        raise ValueError("Could not extract BPE merges.")

    writer.add_tokenizer_model("gpt2")
    writer.add_tokenizer_pre("qwen2")
    writer.add_token_merges(merges)

    vocab = tokenizer.get_vocab()
    tokens = [b""] * len(vocab)
    for token, idx in vocab.items():
        tokens[idx] = token.encode("utf-8", errors="ignore") if isinstance(token, str) else token
    tokens = [t if t != b"" else b"<unk>" for t in tokens]
    writer.add_token_list(tokens)

    types = [1] * len(tokens)                     # 1 = normal, 3 = control
    for sid in tokenizer.all_special_ids:
        if sid < len(tokens):
            types[sid] = 3
    writer.add_token_types(types)
    writer.add_token_scores([0.0] * len(tokens))
    if tokenizer.bos_token_id is not None:
        writer.add_bos_token_id(tokenizer.bos_token_id)
    if tokenizer.eos_token_id is not None:
        writer.add_eos_token_id(tokenizer.eos_token_id)
    if tokenizer.pad_token_id is not None:
        writer.add_pad_token_id(tokenizer.pad_token_id)


def _as_numpy(t: torch.Tensor) -> np.ndarray:
    """Signed views of the unsigned and bf16 tensors, as the reference stores them
    (comp_inference/rans_gguf.py:150-160): ggml has no unsigned or (in this use) bf16 tensor type."""
    view = {torch.bfloat16: torch.int16, torch.uint8: torch.int8, torch.uint16: torch.int16,
            torch.uint32: torch.int32}.get(t.dtype)
    t = t.detach().cpu().contiguous()
    return (t.view(view) if view is not None else t).numpy()


def save_rans_model_gguf(model, tokenizer, output_path: str, model_name: str = None) -> None:
    """Write `model` (its compressible layers already compressed) as one GGUF file with the reference's
    metadata keys and tensor names (comp_inference/rans_gguf.py:111-238): per compressed module
    `<name>.rans_exp_{stream,states,sizes,freqs,cdf}` (or `rans_exp_raw`), `rans_man_raw` (or the
    `rans_man_*` set), `rans_info = [1, numel, exp_compressed, exp_streams, man_compressed, man_streams,
    rank, *shape]` and an fp32 `bias`; every other parameter under its llama.cpp name."""
    cfg = model.config
    w = _Writer(output_path, "qwen3")
    w.add_architecture()
    w.add_block_count(cfg.num_hidden_layers)
    w.add_context_length(getattr(cfg, "max_position_embeddings", 32768))
    w.add_embedding_length(cfg.hidden_size)
    w.add_feed_forward_length(cfg.intermediate_size)
    w.add_head_count(cfg.num_attention_heads)
    w.add_head_count_kv(getattr(cfg, "num_key_value_heads", cfg.num_attention_heads))
    w.add_rope_dimension_count(cfg.hidden_size // cfg.num_attention_heads)
    w.add_rope_freq_base(getattr(cfg, "rope_theta", 1000000.0))
    w.add_layer_norm_rms_eps(getattr(cfg, "rms_norm_eps", getattr(cfg, "layer_norm_epsilon", 1e-6)))
    w.add_string("quantization.method", "rans_bfloat16")
    write_tokenizer(w, tokenizer, model_name)

    for name, module in model.named_modules():
        if getattr(module, "compressed", None) == "rans_bfloat16":
            base = hf_to_gguf_name(name)

            def add(suffix, tensor):
                w.add_tensor(f"{base}.{suffix}", _as_numpy(tensor))

            if hasattr(module, "exponent_compressed_weight"):
                add("rans_exp_stream", module.exponent_compressed_weight)
                add("rans_exp_states", module.exponent_states)
                add("rans_exp_sizes", module.exponent_output_sizes)
                add("rans_exp_freqs", module.exponent_freqs)
                add("rans_exp_cdf", module.exponent_cdf)
                exp_streams, exp_compressed = module.exponent_num_streams, 1
            else:
                add("rans_exp_raw", module.exponent_raw)
                exp_streams, exp_compressed = 0, 0
            if hasattr(module, "mantissa_compressed_weight"):
                add("rans_man_stream", module.mantissa_compressed_weight)
                add("rans_man_states", module.mantissa_states)
                add("rans_man_sizes", module.mantissa_output_sizes)
                add("rans_man_freqs", module.mantissa_freqs)
                add("rans_man_cdf", module.mantissa_cdf)
                man_streams, man_compressed = module.mantissa_num_streams, 1
            else:
                add("rans_man_raw", module.mantissa_raw.flatten())
                man_streams, man_compressed = 0, 0
            shape = list(getattr(module, "input_shape", []) or [])
            if not shape and hasattr(module, "expanded_size"):
                shape = [module.expanded_size]
            info = [1, module.expanded_size, exp_compressed, exp_streams, man_compressed, man_streams,
                    len(shape)] + shape
            add("rans_info", torch.tensor(info, dtype=torch.int32))
            if getattr(module, "bias", None) is not None:
                add("bias", module.bias.float())
        else:
            for pname, param in module.named_parameters(recurse=False):
                if pname == "weight" and hasattr(module, "compressed"):
                    continue
                full = f"{name}.{pname}" if name else pname
                data = param.detach().cpu()
                if data.dtype == torch.bfloat16:
                    data = data.view(torch.int16)
                w.add_tensor(hf_to_gguf_name(full), data.contiguous().numpy())
    w.write()
