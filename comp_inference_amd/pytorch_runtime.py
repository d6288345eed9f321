"""Inference modules that keep their weights compressed, mirroring
comp_inference/pytorch_runtime.py:386-642 of the reference: `RansWorkspace`, `RansLinear`,
`RansLMHead`, `RansEmbedding` (same constructor arguments and buffer names/dtypes, so a package
written by the reference loads by key) and the model loader.
"""
from __future__ import annotations

import json
import os

import torch
import torch.nn as nn

from .embedding_hip import fused_rans_embedding
from .linear_hip import PreparedLinear, fused_rans_linear
from .rans_hip import build_checkpoints, suggest_segments
from .transposed_linear_hip import fused_rans_linear_transposed


class RansWorkspace:
    """Grow-only split-K workspace shared by all layers (comp_inference/pytorch_runtime.py:386-394)."""
    _buffer = None

    @classmethod
    def get_workspace(cls, M, N, split_k, device):
        elements = M * N * split_k
        if cls._buffer is None or cls._buffer.numel() < elements or cls._buffer.device != torch.device(device):
            cls._buffer = torch.zeros(elements * 2, device=device, dtype=torch.bfloat16)
        return cls._buffer[:elements].view(split_k, M, N)


def _register_rans_buffers(mod: nn.Module) -> None:
    # names and dtypes as comp_inference/pytorch_runtime.py:413-424; the slot map is stored as
    # uint8 in every package (comp_inference/rans_saving.py:406-408) and arrives as such
    mod.register_buffer("rans_exp_stream", torch.empty(0, dtype=torch.uint8))
    mod.register_buffer("rans_exp_states", torch.empty(0, dtype=torch.uint32))
    mod.register_buffer("rans_exp_tables", torch.empty(0, dtype=torch.uint32))
    mod.register_buffer("rans_exp_slot_map", torch.empty(0, dtype=torch.uint16))
    mod.register_buffer("rans_exp_tile_offsets", torch.empty(0, dtype=torch.uint32))
    mod.register_buffer("rans_exp_tile_max_lens", torch.empty(0, dtype=torch.uint32))
    mod.register_buffer("rans_man_raw", torch.empty(0, dtype=torch.uint8))
    mod.register_buffer("rans_info", torch.empty(0, dtype=torch.int32))


def _load_from_compressed(mod: nn.Module, src: nn.Module) -> None:
    """Fill the buffers from a module compressed with rans_compress_module_weight."""
    if getattr(src, "exponent_uncoalesced_interleaving", False):
        raise ValueError("the runtime modules take the default (tile-interleaved) format")
    mod.rans_exp_stream = src.exponent_compressed_weight.clone()
    mod.rans_exp_states = src.exponent_states.clone()
    mod.rans_exp_tables = src.exponent_tables.clone()
    mod.rans_exp_slot_map = src.exponent_slot_map.clone()
    mod.rans_exp_tile_offsets = src.exponent_tile_offsets.clone()
    mod.rans_exp_tile_max_lens = src.exponent_tile_max_lens.clone()
    mod.rans_man_raw = src.mantissa_raw.clone()
    mod.tile_k, mod.tile_n = int(src.exponent_tile_height), int(src.exponent_tile_width)


def _version_of(t: torch.Tensor) -> int:
    """Version counter of a tensor for the cache keys below; tensors made under torch.inference_mode() (a model
    loaded or moved inside it) do not track one and cannot be updated in place either: 0."""
    return 0 if t.is_inference() else t._version


def _cached_checkpoints(mod: nn.Module, device, shape, segments: int):
    """(checkpoints, segments) of `mod`'s compressed weight as it lies on `device`: built on first use from
    the stream (one pass of the decoder) and kept beside it; derived data, not part of the saved state."""
    cached = getattr(mod, "_ckpt_cache", None)
    st = mod.rans_exp_stream
    key = ((st.data_ptr(), st.numel(), _version_of(st)), device, segments)  # (a reload swaps the storage, not the tensor)
    if cached is not None and cached[0] == key:
        return cached[1], cached[2]
    ck = None
    if segments > 1:
        ck = build_checkpoints(mod.rans_exp_stream.to(device), mod.rans_exp_states.to(device),
                               mod.rans_exp_tables.to(device), mod.rans_exp_slot_map.to(device), shape,
                               mod.rans_exp_tile_offsets.to(device), mod.rans_exp_tile_max_lens.to(device),
                               mod.tile_k, mod.tile_n, segments)
    mod._ckpt_cache = (key, ck, segments if ck is not None else 1)
    return mod._ckpt_cache[1], mod._ckpt_cache[2]


class RansLinear(nn.Module):
    """comp_inference/pytorch_runtime.py:397-459.  Weight stored as [K=in, N=out]."""

    def __init__(self, in_features: int, out_features: int, tile_k: int = 1024, tile_n: int = 32,
                 split_k: int = 1, has_bias: bool = False):
        super().__init__()
        self.in_features, self.out_features = in_features, out_features
        self.tile_k, self.tile_n, self.split_k = tile_k, tile_n, split_k
        _register_rans_buffers(self)
        if has_bias:
            self.register_buffer("bias", torch.empty(out_features, dtype=torch.bfloat16))
        else:
            self.bias = None

    @classmethod
    def from_compressed(cls, src: nn.Module, bias=None, split_k: int = 1) -> "RansLinear":
        K, N = src.input_shape
        mod = cls(K, N, split_k=split_k, has_bias=bias is not None)
        _load_from_compressed(mod, src)
        if bias is not None:
            mod.bias = bias.detach().to(torch.bfloat16).clone()
        return mod

    # Weights with few tiles are bound by the length of one stream's decode chain; decoder checkpoints cut
    # every stream into segments that decode side by side.  `auto`: as many segments as the library
    # suggests for the shape; an int fixes them; 1 switches the index off.
    segments = "auto"

    def _checkpoints(self, device):
        shape = (self.in_features, self.out_features)
        segs = suggest_segments(shape, self.tile_k, self.tile_n) if self.segments == "auto" else int(self.segments)
        return _cached_checkpoints(self, device, shape, segs)

    def _buffers_key(self):
        """What the prepared call was made from: storage, length and version of every buffer, so that a reload
        that swaps `tensor.data` under an unchanged tensor object (the loader's own idiom) or an in-place update
        is noticed."""
        ts = (self.rans_exp_stream, self.rans_exp_states, self.rans_man_raw, self.bias)  # (a reload replaces them all)
        return tuple((t.data_ptr(), t.numel(), _version_of(t)) if t is not None else None for t in ts)

    # True: the buffers are converted once per device and the result is kept (PreparedLinear; a module whose buffers
    # live on the host then holds a device copy for good).  False: the reference's way -- every call moves the buffers
    # to the input's device and lets go of them afterwards (comp_inference/pytorch_runtime.py:440-459), so a model
    # larger than the GPU can stay on the host; no decoder checkpoints then (they would be resident derived data).
    resident = True

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        device = x.device
        if not self.resident:
            from .linear_hip import fused_rans_linear

            to = lambda t: t.to(device, non_blocking=True)  # noqa: E731
            return fused_rans_linear(
                x=x, compressed_data=to(self.rans_exp_stream), initial_states=to(self.rans_exp_states),
                tables=to(self.rans_exp_tables), slot_map=to(self.rans_exp_slot_map),
                weight_shape=(self.in_features, self.out_features), tile_offsets=to(self.rans_exp_tile_offsets),
                tile_max_lens=to(self.rans_exp_tile_max_lens), tile_k=self.tile_k, tile_n=self.tile_n,
                mantissas=to(self.rans_man_raw), bias=None if self.bias is None else to(self.bias), SPLIT_K=self.split_k)
        prepared = getattr(self, "_prepared", None)
        key = (self._buffers_key(), device, self.segments)
        if prepared is None or prepared[0] != key:
            from . import _lib

            _lib.require_device(x)
            checkpoints, segments = self._checkpoints(device)
            call = PreparedLinear(device, self.rans_exp_stream, self.rans_exp_states, self.rans_exp_tables,
                                  self.rans_exp_slot_map, (self.in_features, self.out_features),
                                  self.rans_exp_tile_offsets, self.rans_exp_tile_max_lens, self.tile_k, self.tile_n,
                                  self.rans_man_raw, self.bias, checkpoints, segments)
            prepared = self._prepared = (key, call)
        return prepared[1](x)


class RansLMHead(nn.Module):
    """comp_inference/pytorch_runtime.py:462-505.  Weight stored as [out=vocab, in=hidden]: the
    embedding table's layout, so a tied head shares the table's buffers."""

    def __init__(self, in_features: int, out_features: int, tile_k: int = 1024, tile_n: int = 32):
        super().__init__()
        self.in_features, self.out_features = in_features, out_features
        self.tile_k, self.tile_n = tile_k, tile_n
        _register_rans_buffers(self)

    @classmethod
    def from_compressed(cls, src: nn.Module) -> "RansLMHead":
        V, H = src.input_shape
        mod = cls(H, V)
        _load_from_compressed(mod, src)
        return mod

    def tie_to(self, emb: "RansEmbedding") -> None:
        for name in ("rans_exp_stream", "rans_exp_states", "rans_exp_tables", "rans_exp_slot_map",
                     "rans_exp_tile_offsets", "rans_exp_tile_max_lens", "rans_man_raw", "rans_info"):
            setattr(self, name, getattr(emb, name))
        self.tile_k, self.tile_n = emb.tile_k, emb.tile_n
        self.tied_to_embedding = True

    # Derived data kept beside the weight, built on first use: decoder checkpoints (so that one row of x runs on
    # sixteen wavefronts per CU), the largest window an item reads, the slot table in its LDS form.  `auto`: as many
    # segments as the library suggests for the shape; an int fixes them; 1 (the default) switches the index off.
    segments = 1

    def _derived(self, device):
        import ctypes as C

        from . import _lib

        shape = (self.out_features, self.in_features)
        segs = suggest_segments(shape, self.tile_k, self.tile_n) if self.segments == "auto" else int(self.segments)
        ck, segs = _cached_checkpoints(self, device, shape, segs)
        cached = getattr(self, "_derived_cache", None)
        key = (self._ckpt_cache[0], segs)
        if cached is not None and cached[0] == key:
            return ck, segs, cached[1], cached[2]
        max_rows, table = 0, None
        if segs > 1 and self.tile_n == 32:
            t = [b.to(device) for b in (self.rans_exp_stream, self.rans_exp_states, self.rans_exp_tables, self.rans_exp_slot_map,
                                        self.rans_exp_tile_offsets, self.rans_exp_tile_max_lens)]
            t = [_lib.as_u8(t[0], device), _lib.as_u32(t[1], device), _lib.as_u32(t[2], device), _lib.as_u8(t[3], device),
                 _lib.as_u32(t[4], device), _lib.as_u32(t[5], device)]
            table = torch.empty(_lib.SLOT_TABLE_BYTES, dtype=torch.uint8, device=device)
            rows = torch.zeros(1, dtype=torch.int32, device=device)
            w = _lib.tiled_weight(shape[0], shape[1], self.tile_k, self.tile_n, t[0], t[1], t[2], t[3], t[4], t[5], None, ck, segs)
            with torch.cuda.device(device):
                _lib.check(_lib.lib().ci_build_slot_table(_lib.ptr(t[2]), _lib.ptr(t[3]), _lib.ptr(table),
                                                          C.c_size_t(_lib.SLOT_TABLE_BYTES), _lib.stream_handle(device)))
                _lib.check(_lib.lib().ci_max_window_rows(C.byref(w), _lib.ptr(rows), _lib.stream_handle(device)))
            max_rows = int(rows.item())
        self._derived_cache = (key, max_rows, table)
        return ck, segs, max_rows, table

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        device = x.device
        ck, segs, max_rows, table = self._derived(device)
        return fused_rans_linear_transposed(
            x=x, checkpoints=ck, segments=segs, max_window_rows=max_rows, slot_table=table,
            compressed_data=self.rans_exp_stream.to(device, non_blocking=True),
            initial_states=self.rans_exp_states.to(device, non_blocking=True),
            tables=self.rans_exp_tables.to(device, non_blocking=True),
            slot_map=self.rans_exp_slot_map.to(device, non_blocking=True),
            weight_shape=(self.out_features, self.in_features),
            tile_offsets=self.rans_exp_tile_offsets.to(device, non_blocking=True),
            tile_max_lens=self.rans_exp_tile_max_lens.to(device, non_blocking=True),
            tile_n=self.tile_n, tile_k=self.tile_k,
            mantissas=self.rans_man_raw.to(device, non_blocking=True),
            workspace=None, SPLIT_K=1, bias=None)


class RansEmbedding(nn.Module):
    """comp_inference/pytorch_runtime.py:508-549.  Table stored as [vocab, dim], not transposed."""

    def __init__(self, num_embeddings: int, embedding_dim: int, tile_k: int = 1024, tile_n: int = 32):
        super().__init__()
        self.num_embeddings, self.embedding_dim = num_embeddings, embedding_dim
        self.tile_k, self.tile_n = tile_k, tile_n
        _register_rans_buffers(self)

    @classmethod
    def from_compressed(cls, src: nn.Module) -> "RansEmbedding":
        V, H = src.input_shape
        mod = cls(V, H)
        _load_from_compressed(mod, src)
        return mod

    # Decoder checkpoints every 64 rows (8 segments of a 512-row stream): a looked-up row then costs at most
    # 64 decode steps instead of 512, for an index of 8 % of the compressed table.  1 switches it off.
    segments = "auto"

    def _checkpoints(self, device):
        half = self.tile_k // 2
        segs = int(self.segments) if self.segments != "auto" else \
            (max(1, half // 64) if self.tile_n == 32 and half % 64 == 0 else 1)
        return _cached_checkpoints(self, device, (self.num_embeddings, self.embedding_dim), segs)

    # The gather on sixteen wavefronts per CU (needs checkpoints and the slot table kept beside the table, built on
    # first use).  Off until that kernel has been measured.
    sixteen_wavefronts = False

    def _slot_table(self, device):
        from .rans_hip import build_slot_table

        t, m = self.rans_exp_tables, self.rans_exp_slot_map
        key = (str(device), t.data_ptr(), _version_of(t), m.data_ptr(), _version_of(m))
        cached = getattr(self, "_slot_table_cache", None)
        if cached is None or cached[0] != key:
            cached = (key, build_slot_table(t, m, device))
            self._slot_table_cache = cached
        return cached[1]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        device = x.device
        checkpoints, segments = self._checkpoints(device)
        return fused_rans_embedding(
            x=x,
            checkpoints=checkpoints, segments=segments,
            slot_table=self._slot_table(device) if self.sixteen_wavefronts and segments > 1 else None,
            compressed_data=self.rans_exp_stream.to(device, non_blocking=True),
            initial_states=self.rans_exp_states.to(device, non_blocking=True),
            tables=self.rans_exp_tables.to(device, non_blocking=True),
            slot_map=self.rans_exp_slot_map.to(device, non_blocking=True),
            weight_shape=(self.num_embeddings, self.embedding_dim),
            tile_offsets=self.rans_exp_tile_offsets.to(device, non_blocking=True),
            tile_max_lens=self.rans_exp_tile_max_lens.to(device, non_blocking=True),
            tile_k=self.tile_k, tile_n=self.tile_n,
            mantissas=self.rans_man_raw.to(device, non_blocking=True))


def swap_in_rans_modules(model: nn.Module, state_dict: dict, quant_config: dict | None = None,
                         split_k: int = 1) -> nn.Module:
    """Replace every nn.Linear / nn.Embedding / lm_head whose `<name>.rans_exp_stream` key exists in
    `state_dict` by its compressed counterpart and assign all matching tensors
    (comp_inference/pytorch_runtime.py:563-637).  Works on any already constructed model, so no
    network access is needed."""
    quant_config = quant_config or {}
    layer_configs = quant_config.get("layer_configs", {})
    default_th = quant_config.get("default_tile_height", 1024)
    default_tw = quant_config.get("default_tile_width", 32)

    def tile_of(name):
        cfg = layer_configs.get(name, {})
        return cfg.get("tile_height", default_th), cfg.get("tile_width", default_tw)

    replacements = []
    for name, module in model.named_modules():
        if "lm_head" in name or isinstance(module, (RansLinear, RansEmbedding, RansLMHead)):
            continue
        if f"{name}.rans_exp_stream" not in state_dict:
            continue
        th, tw = tile_of(name)
        if isinstance(module, nn.Linear):
            replacements.append((name, RansLinear(module.in_features, module.out_features, th, tw, split_k,
                                                  module.bias is not None)))
        elif isinstance(module, nn.Embedding):
            replacements.append((name, RansEmbedding(module.num_embeddings, module.embedding_dim, th, tw)))
    for name, new_layer in replacements:
        parent_name, _, child = name.rpartition(".")
        parent = model.get_submodule(parent_name) if parent_name else model
        setattr(parent, child, new_layer)
    if hasattr(model, "lm_head") and "lm_head.rans_exp_stream" in state_dict:
        th, tw = tile_of("lm_head")
        model.lm_head = RansLMHead(model.lm_head.in_features, model.lm_head.out_features, tile_k=th, tile_n=tw)
    elif hasattr(model, "lm_head") and not any(k in state_dict for k in ("lm_head.weight", "model.lm_head.weight")):
        # A package written with a tied head holds neither lm_head.weight nor a compressed head: the head is the
        # embedding table.  The reference gets there through from_pretrained's own tying; a model built from its
        # config alone (or handed in) would keep a randomly initialised head once the embedding has been
        # replaced, so the head is tied to the compressed table here -- or the load fails.
        emb = model.get_input_embeddings() if hasattr(model, "get_input_embeddings") else None
        if isinstance(emb, RansEmbedding):
            head = RansLMHead(model.lm_head.in_features, model.lm_head.out_features, tile_k=emb.tile_k, tile_n=emb.tile_n)
            head.tie_to(emb)
            model.lm_head = head
        elif isinstance(emb, nn.Embedding) and isinstance(model.lm_head, nn.Linear):
            model.lm_head.weight = emb.weight
        else:
            raise RuntimeError("the file holds no lm_head weights and the model has no embedding to tie the head to")

    targets = dict(model.named_buffers())
    targets.update(dict(model.named_parameters()))
    for name, tensor in targets.items():
        if name in state_dict:
            tensor.data = state_dict[name].contiguous()
    return model


def load_compressed_model_with_auto_model(model_id: str, safetensors_path: str, split_k: int = 1,
                                          compile_model: bool = False, model: nn.Module | None = None):
    """comp_inference/pytorch_runtime.py:552-642.  `model_id` may be a local directory holding
    config.json (the model is then built from the config alone, no download); pass `model` to
    swap modules in a model built elsewhere."""
    from safetensors.torch import load_file

    quant_config = {}
    if model is None:
        from transformers import AutoConfig, AutoModelForCausalLM

        if os.path.isdir(model_id):
            config = AutoConfig.from_pretrained(model_id)
            model = AutoModelForCausalLM.from_config(config, torch_dtype=torch.bfloat16)
        else:
            model = AutoModelForCausalLM.from_pretrained(model_id, torch_dtype=torch.bfloat16)
        quant_config = getattr(model.config, "quantization_config", {}) or {}
        if not isinstance(quant_config, dict):
            quant_config = quant_config.to_dict()
    else:
        cfg_path = os.path.join(os.path.dirname(safetensors_path), "config.json")
        if os.path.exists(cfg_path):
            quant_config = json.load(open(cfg_path)).get("quantization_config", {})
    state_dict = load_file(safetensors_path, device="cpu")
    model = swap_in_rans_modules(model, state_dict, quant_config, split_k)
    model = model.cuda()
    # (moving a module gives each of its buffers a tensor of its own: a head tied to the table is tied again,
    # so that the table is on the GPU once)
    head, emb = getattr(model, "lm_head", None), model.get_input_embeddings() if hasattr(model, "get_input_embeddings") else None
    if isinstance(head, RansLMHead) and getattr(head, "tied_to_embedding", False) and isinstance(emb, RansEmbedding):
        head.tie_to(emb)
    return model
