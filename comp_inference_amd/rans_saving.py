"""safetensors package of a compressed model: tensor names, dtypes and the `rans_info` record of
comp_inference/rans_saving.py:352-481, the `quantization_config` block of :19-109, the file-level
metadata of :238-242.
"""
from __future__ import annotations

import json
import os

import torch
from safetensors.torch import save_file

RANS_INFO_FIELDS = ("version", "numel", "exp_compressed", "exp_streams", "man_compressed", "man_streams",
                    "rank", "num_tiles_n", "num_tiles_k", "tile_height", "tile_width")


def _cpu(t: torch.Tensor, dtype) -> torch.Tensor:
    t = t.detach().cpu()
    if t.dtype != dtype:
        t = t.to(torch.int64).to(dtype) if dtype == torch.uint32 else t.to(dtype)
    return t.contiguous()


def rans_tensors_for_module(base_name: str, module) -> dict:
    """Tensors of one compressed module under `<base_name>rans_*` keys
    (comp_inference/rans_saving.py:352-481); base_name ends with '.'."""
    out = {}
    p = base_name
    out[p + "rans_exp_stream"] = _cpu(module.exponent_compressed_weight, torch.uint8)
    out[p + "rans_exp_states"] = _cpu(module.exponent_states, torch.uint32)
    out[p + "rans_exp_tables"] = _cpu(module.exponent_tables, torch.uint32)
    out[p + "rans_exp_slot_map"] = _cpu(module.exponent_slot_map, torch.uint8)
    if getattr(module, "exponent_uncoalesced_interleaving", False):
        out[p + "rans_exp_stream_offsets"] = _cpu(module.exponent_stream_offsets, torch.uint32)
    else:
        out[p + "rans_exp_tile_offsets"] = _cpu(module.exponent_tile_offsets, torch.uint32)
        out[p + "rans_exp_tile_max_lens"] = _cpu(module.exponent_tile_max_lens, torch.uint32)
    out[p + "rans_man_raw"] = _cpu(module.mantissa_raw, torch.uint8)
    shape = list(getattr(module, "input_shape", [module.expanded_size]))
    info = [1, module.expanded_size, 1, module.exponent_num_streams, 0, 0, len(shape),
            module.exponent_num_tiles_n, module.exponent_num_tiles_k, module.exponent_tile_height,
            module.exponent_tile_width] + shape
    out[p + "rans_info"] = torch.tensor(info, dtype=torch.int32)
    bias = getattr(module, "bias", None)
    if bias is not None:
        out[p + "bias"] = bias.detach().cpu()
    return out


def parse_rans_info(info: torch.Tensor) -> dict:
    vals = [int(v) for v in info.tolist()]
    d = dict(zip(RANS_INFO_FIELDS, vals))
    d["shape"] = vals[len(RANS_INFO_FIELDS):len(RANS_INFO_FIELDS) + d["rank"]]
    return d


def collect_tensors(model, tied_lm_head: bool = False) -> dict:
    tensors, handled = {}, set()
    if tied_lm_head:
        handled.update({"lm_head.weight", "model.lm_head.weight"})
    for name, module in model.named_modules():
        if getattr(module, "compressed", None) == "rans_bfloat16":
            # (a compressed lm_head keeps its tensors also when the head is tied, as in
            # comp_inference/rans_saving.py:193-227: only the plain lm_head.weight is dropped)
            tensors.update(rans_tensors_for_module(name + ".", module))
            handled.update({f"{name}.weight", f"{name}.bias"})
    for pname, param in model.named_parameters():
        if pname not in handled:
            tensors[pname] = param.data.cpu().contiguous()
    return tensors


def pack_and_save_tensors(model, output_path: str, fuse: bool = False, tied_lm_head: bool = False):
    """comp_inference/rans_saving.py:177-245."""
    tensors = collect_tensors(model, tied_lm_head)
    metadata = {"format": "pt", "compression_method": "rans_bfloat16", "fused_projections": str(fuse)}
    save_file(tensors, output_path, metadata=metadata)
    return tensors


def quantization_config_for(model, fuse: bool = False, tied_lm_head: bool = False) -> dict:
    """comp_inference/rans_saving.py:33-98."""
    layer_configs = {}
    for name, module in model.named_modules():
        if tied_lm_head and "lm_head" in name:
            continue
        if getattr(module, "compressed", None) != "rans_bfloat16":
            continue
        if fuse:
            if "gate_proj" in name:
                name = name.replace("gate_proj", "gate_up_proj")
            elif "q_proj" in name:
                name = name.replace("q_proj", "qkv_proj")
        layer_configs[name] = {
            "tile_height": int(getattr(module, "exponent_tile_height", 1024)),
            "tile_width": int(getattr(module, "exponent_tile_width", 32)),
            "uncoalesced_interleaving": bool(getattr(module, "exponent_uncoalesced_interleaving", False)),
        }
    return {"quant_method": "rans", "compression": "rans_bfloat16", "layer_configs": layer_configs,
            "default_tile_height": 1024, "default_tile_width": 32, "fused_projections": fuse}


def save_rans_model_package(model, tokenizer, output_dir: str, fuse: bool = False, tied_lm_head: bool = False):
    """config.json (+ tokenizer) + model.safetensors (comp_inference/rans_saving.py:19-109).
    As in the reference, an unfused package goes to `<output_dir>_unfused`."""
    if not fuse:
        output_dir = output_dir + "_unfused"
    os.makedirs(output_dir, exist_ok=True)
    qc = quantization_config_for(model, fuse, tied_lm_head)
    config = getattr(model, "config", None)
    if config is not None and hasattr(config, "save_pretrained"):
        config.quantization_config = qc
        config.save_pretrained(output_dir)
    else:
        cfg = dict(config) if isinstance(config, dict) else {}
        cfg["quantization_config"] = qc
        with open(os.path.join(output_dir, "config.json"), "w") as f:
            json.dump(cfg, f, indent=2)
    if tokenizer is not None:
        tokenizer.save_pretrained(output_dir)
    path = os.path.join(output_dir, "model.safetensors")
    pack_and_save_tensors(model, path, fuse=fuse, tied_lm_head=tied_lm_head)
    return output_dir


def _load_rans_layer(module, prefix: str, f, keys) -> None:
    """Attributes of one compressed module from its `<prefix>.rans_*` tensors
    (comp_inference/rans_saving.py:542-656).  Unlike the reference, tensors the writer does not store
    (`rans_exp_sizes`) are optional, and the tile arrays are loaded whenever the file has them (the
    reference reads them only into attributes that already exist, :599-613)."""
    info = parse_rans_info(f.get_tensor(f"{prefix}.rans_info"))
    module.compressed = "rans_bfloat16"
    module.expanded_size = info["numel"]
    module.input_shape = list(info["shape"])
    module.tile_height = module.exponent_tile_height = info["tile_height"]
    module.tile_width = module.exponent_tile_width = info["tile_width"]
    if info["exp_compressed"] <= 0:
        raise ValueError(f"Corrupt file: {prefix} has no coded exponent plane (a raw one is never written)")
    module.exponent_compressed_weight = f.get_tensor(f"{prefix}.rans_exp_stream")
    module.exponent_states = f.get_tensor(f"{prefix}.rans_exp_states")
    if f"{prefix}.rans_exp_sizes" in keys:
        module.exponent_output_sizes = f.get_tensor(f"{prefix}.rans_exp_sizes")
    module.exponent_tables = f.get_tensor(f"{prefix}.rans_exp_tables")
    module.exponent_slot_map = f.get_tensor(f"{prefix}.rans_exp_slot_map")
    module.exponent_num_streams = info["exp_streams"]
    module.exponent_stream_size = module.exponent_total_stream_size = module.exponent_compressed_weight.numel()
    module.exponent_num_tiles_n, module.exponent_num_tiles_k = info["num_tiles_n"], info["num_tiles_k"]
    dense = f"{prefix}.rans_exp_stream_offsets" in keys
    module.exponent_uncoalesced_interleaving = dense
    if dense:
        module.exponent_stream_offsets = f.get_tensor(f"{prefix}.rans_exp_stream_offsets")
    else:
        module.exponent_tile_offsets = f.get_tensor(f"{prefix}.rans_exp_tile_offsets")
        module.exponent_tile_max_lens = f.get_tensor(f"{prefix}.rans_exp_tile_max_lens")
    if f"{prefix}.rans_man_raw" not in keys:
        raise ValueError(f"Corrupt file: {prefix} marked uncompressed mantissa but raw data missing.")
    module.mantissa_raw = f.get_tensor(f"{prefix}.rans_man_raw")
    if f"{prefix}.bias" in keys and getattr(module, "bias", None) is not None:
        module.bias.data = f.get_tensor(f"{prefix}.bias")
    if hasattr(module, "weight"):
        del module.weight  # the skeleton's weight; a forward before decompression must fail loudly


def load_compressed_model(model, safetensors_path: str, device="cpu"):
    """Load a compressed safetensors file into an initialised model skeleton: compressed modules
    get their `exponent_*` / `mantissa_raw` attributes back (ready for rans_decompress_module_weight
    or the Rans* runtime modules), everything else its parameters
    (comp_inference/rans_saving.py:497-539)."""
    from safetensors import safe_open

    loaded = 0
    with safe_open(safetensors_path, framework="pt", device=str(device)) as f:
        keys = set(f.keys())
        for name, module in model.named_modules():
            if f"{name}.rans_info" in keys:
                _load_rans_layer(module, name, f, keys)
                loaded += 1
                continue
            for pname, param in module.named_parameters(recurse=False):
                full = f"{name}.{pname}" if name else pname
                if full in keys:
                    tensor = f.get_tensor(full)
                    if param.shape != tensor.shape:
                        print(f"Warning: Shape mismatch for {full}. Expected {param.shape}, got {tensor.shape}")
                    param.data = tensor
    print(f"Model loaded. {loaded} layers are compressed.")
    return model
