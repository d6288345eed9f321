#!/usr/bin/env python3
"""Batch-1 greedy decode of a Llama-3-8B-shaped random-init decoder whose linear and embedding
weights are rANS-compressed (RansLinear / RansEmbedding / RansLMHead), against the same decoder on
the decompressed bf16 weights -- once through torch.matmul (hipBLASLt) and once through the fused
kernels' own contraction order applied to the plain weights (`plain_linear_same_order`), the run
whose generated ids the compressed model must reproduce exactly.

  python bench_model.py [--layers 32] [--prompt 128] [--new 256] [--tile-k 1024] [--gen cpu|cuda]

Prints one JSON object: tokens per second of the compressed model (eager launches and one HIP
graph replay per token), of the bf16 reference, and how the generated ids and logits compare.

Shape: hidden 4096, FFN 14336 SwiGLU, 32 query / 8 KV heads of 128, vocabulary 128256, RMSNorm,
RoPE theta 500000.  Weights bf16 N(0, 0.02) from seed 5 in module order (embedding; per layer q, k, v,
o, gate, up, down; lm_head), norm weights 1; q/k/v and gate/up are compressed as fused projections
(comp_inference/comp_inference.py:242-341).  Prompt: uniform random ids from seed 6.
Everything except the linear / embedding / head operators is the same torch code in both models.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch
import torch.nn.functional as F

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)


class Shape:
    hidden, ffn, heads, kv_heads, head_dim, vocab = 4096, 14336, 32, 8, 128, 128256
    theta, eps = 500000.0, 1e-5


def log(msg):
    print(msg, file=sys.stderr, flush=True)


def rmsnorm(x, eps):
    return F.rms_norm(x, (x.shape[-1],), eps=eps)  # norm weights are 1


def rope(x, cos, sin):
    """x [T, heads, head_dim]; cos/sin [T, head_dim] (HF rotate-half convention)."""
    xf = x.float()
    h = xf.shape[-1] // 2
    rot = torch.cat((-xf[..., h:], xf[..., :h]), dim=-1)
    return (xf * cos[:, None, :] + rot * sin[:, None, :]).to(torch.bfloat16)


class Dense:
    """x @ W for a decompressed [K, N] bf16 weight: the reference operator."""

    def __init__(self, w_kn):
        self.w = w_kn

    def __call__(self, x):
        return torch.matmul(x, self.w)


class PlainSameOrder:
    """x @ W for a decompressed [K, N] bf16 weight through the fused kernel's contraction order: what the
    compressed operator computes if, and only if, it reconstructs every weight bit."""

    def __init__(self, w_kn, tile_k, tile_n):
        import comp_inference_amd as ci

        self.w, self.tile_k, self.tile_n = w_kn, tile_k, tile_n
        # the compressed operator splits every stream into this many segments (decoder checkpoints),
        # which is also how its contraction is split into partial sums
        self.segments = ci.suggest_segments(tuple(w_kn.shape), tile_k, tile_n)

    def __call__(self, x):
        import comp_inference_amd as ci

        return ci.plain_linear_same_order(x, self.w, tile_k=self.tile_k, tile_n=self.tile_n, segments=self.segments)


class Decoder:
    """The decoder over a set of operators: embed(ids) -> [T, H]; per layer qkv, o, gate_up, down;
    head(x) -> [T, V].  Static KV cache so that one decode step has fixed shapes."""

    def __init__(self, ops, n_layers, max_len, dev):
        s = Shape
        self.ops, self.L, self.max_len, self.dev = ops, n_layers, max_len, dev
        self.k = torch.zeros(n_layers, s.kv_heads, max_len, s.head_dim, dtype=torch.bfloat16, device=dev)
        self.v = torch.zeros_like(self.k)
        inv = 1.0 / (s.theta ** (torch.arange(0, s.head_dim, 2, dtype=torch.float32, device=dev) / s.head_dim))
        ang = torch.arange(max_len, dtype=torch.float32, device=dev)[:, None] * inv[None, :]
        self.cos = torch.cat((ang.cos(), ang.cos()), dim=-1)
        self.sin = torch.cat((ang.sin(), ang.sin()), dim=-1)
        self.positions = torch.arange(max_len, device=dev)

    def _layer(self, l, h, pos, T):
        """h [T, H]; pos int64 [T] (device).  Attention reads the whole cache, masked by position."""
        s = Shape
        qkv = self.ops["qkv"][l](rmsnorm(h, s.eps))
        qkv = qkv.view(T, s.heads + 2 * s.kv_heads, s.head_dim)
        qk = rope(qkv[:, :s.heads + s.kv_heads], self.cos.index_select(0, pos), self.sin.index_select(0, pos))
        self.k[l].index_copy_(1, pos, qk[:, s.heads:].transpose(0, 1))
        self.v[l].index_copy_(1, pos, qkv[:, s.heads + s.kv_heads:].transpose(0, 1))
        allowed = self.positions[None, :] <= pos[:, None]                        # [T, max_len]
        ctx = F.scaled_dot_product_attention(qk[:, :s.heads].transpose(0, 1)[None], self.k[l][None], self.v[l][None],
                                             attn_mask=allowed[None, None], enable_gqa=True)[0]  # [heads, T, d]
        h = h + self.ops["o"][l](ctx.transpose(0, 1).reshape(T, s.heads * s.head_dim))
        gu = self.ops["gate_up"][l](rmsnorm(h, s.eps))
        gate, up = gu.split((s.ffn, s.ffn), dim=-1)
        return h + self.ops["down"][l](F.silu(gate) * up)

    def forward(self, ids, pos):
        """ids, pos int64 [T] -> logits of the last position [V] (fp32)."""
        T = ids.shape[0]
        h = self.ops["embed"](ids)
        for l in range(self.L):
            h = self._layer(l, h, pos, T)
        return self.ops["head"](rmsnorm(h[-1:], Shape.eps)).float().view(-1)


def generate(dec: Decoder, prompt, n_new, use_graph):
    """Greedy decode; returns (ids list, seconds for the n_new decode steps, prefill excluded)."""
    dev = dec.dev
    P = prompt.numel()
    logits = dec.forward(prompt, torch.arange(P, device=dev))
    tok = torch.argmax(logits).view(1)
    pos = torch.full((1,), P, dtype=torch.int64, device=dev)
    out = torch.zeros(n_new, dtype=torch.int64, device=dev)
    slot = torch.zeros(1, dtype=torch.int64, device=dev)

    def step():
        out.index_copy_(0, slot, tok)
        nxt = torch.argmax(dec.forward(tok, pos)).view(1)
        tok.copy_(nxt)
        pos.add_(1)
        slot.add_(1)

    if not use_graph:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n_new):
            step()
        torch.cuda.synchronize()
        return out.tolist(), time.perf_counter() - t0

    # One HIP graph replay per token.  State (tok, pos, slot, KV cache) lives in static tensors; the
    # capture itself does not execute, so the captured step is the first decode step.
    saved = (tok.clone(), pos.clone(), slot.clone())
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()  # warm-up on the side stream (allocations, kernel attributes)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    tok.copy_(saved[0]); pos.copy_(saved[1]); slot.copy_(saved[2])
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n_new):
        graph.replay()
    torch.cuda.synchronize()
    return out.tolist(), time.perf_counter() - t0


def teacher_forced(dec: Decoder, prompt, ids):
    """Logits [len(ids), V] of every decode step when the given ids are fed, whatever the model itself
    would have chosen: the comparison that one flipped argmax does not derail."""
    dev = dec.dev
    P = prompt.numel()
    rows = [dec.forward(prompt, torch.arange(P, device=dev))]
    for t, tok in enumerate(ids[:-1]):
        rows.append(dec.forward(torch.tensor([tok], device=dev), torch.tensor([P + t], device=dev)))
    return torch.stack(rows)


def build(n_layers, dev, tile_k, tile_n, gen):
    """Draw the weights (seed 5, module order), compress them, and keep a decompressed bf16 copy.
    Returns (compressed ops, dense ops through torch.matmul, dense ops in the fused kernels' order, byte counts)."""
    import comp_inference_amd as ci
    from comp_inference_amd.pytorch_runtime import RansEmbedding, RansLinear, RansLMHead

    s = Shape
    g = torch.Generator(gen).manual_seed(5)

    def draw(o, i):
        return (torch.randn(o, i, generator=g, dtype=torch.float32, device=gen) * 0.02).to(torch.bfloat16).to(dev)

    sizes = {"compressed": 0, "bf16": 0}

    def fill(mod, w_kn):
        exp, man = ci.extract_exp_and_mantissa(w_kn)
        f, c = ci.get_rans_lut(exp)
        r = ci.ccore.RansManager(exp.numel()).compress_tiled(exp, f, c, tile_k, tile_n)
        mod.rans_exp_stream = r.stream.to(dev)
        mod.rans_exp_states = r.states.to(dev)
        mod.rans_exp_tables = r.tables.to(dev)
        mod.rans_exp_slot_map = r.slot_map.to(dev)
        mod.rans_exp_tile_offsets = r.tile_offsets.to(dev)
        mod.rans_exp_tile_max_lens = r.tile_max_lens.to(dev)
        mod.rans_man_raw = ci.interleave_mantissas(man, tile_k, tile_n).contiguous().view(-1).to(dev)
        # the bf16 copy comes from the compressed form, so both models hold the same weight bits
        dense = ci.rans_decomp_tiled(mod.rans_exp_stream, mod.rans_exp_states, mod.rans_exp_tables,
                                     mod.rans_exp_slot_map, tuple(w_kn.shape), mod.rans_exp_tile_offsets,
                                     mod.rans_exp_tile_max_lens, tile_k=tile_k, tile_n=tile_n,
                                     mantissas=mod.rans_man_raw)
        assert torch.equal(dense.view(torch.int16), w_kn.view(torch.int16)), "weight does not round-trip"
        sizes["compressed"] += mod.rans_exp_stream.numel() + mod.rans_man_raw.numel() + 4 * mod.rans_exp_states.numel()
        sizes["bf16"] += 2 * w_kn.numel()
        return dense

    def linear(w_out_in):
        w_kn = w_out_in.t().contiguous()
        mod = RansLinear(w_kn.shape[0], w_kn.shape[1], tile_k=tile_k, tile_n=tile_n)
        dense = fill(mod, w_kn)
        return mod, Dense(dense), PlainSameOrder(dense, tile_k, tile_n)

    comp = {"qkv": [], "o": [], "gate_up": [], "down": []}
    ref = {"qkv": [], "o": [], "gate_up": [], "down": []}
    same = {"qkv": [], "o": [], "gate_up": [], "down": []}
    t0 = time.time()
    table = draw(s.vocab, s.hidden)
    emb = RansEmbedding(s.vocab, s.hidden, tile_k=tile_k, tile_n=tile_n)
    table_dense = fill(emb, table)
    comp["embed"], ref["embed"] = emb, (lambda ids, t=table_dense: t.index_select(0, ids))
    same["embed"] = ref["embed"]
    del table
    for l in range(n_layers):
        q, k, v = draw(s.heads * s.head_dim, s.hidden), draw(s.kv_heads * s.head_dim, s.hidden), \
            draw(s.kv_heads * s.head_dim, s.hidden)
        o = draw(s.hidden, s.heads * s.head_dim)
        gate, up = draw(s.ffn, s.hidden), draw(s.ffn, s.hidden)
        down = draw(s.hidden, s.ffn)
        for name, w in (("qkv", torch.cat((q, k, v), 0)), ("o", o), ("gate_up", torch.cat((gate, up), 0)),
                        ("down", down)):
            m, d, p = linear(w)
            comp[name].append(m)
            ref[name].append(d)
            same[name].append(p)
        if l % 4 == 3 or l == n_layers - 1:
            log(f"  layer {l + 1}/{n_layers} compressed ({time.time() - t0:.0f} s)")
    head_w = draw(s.vocab, s.hidden)                   # [V, H]: the head keeps the table's orientation
    head = RansLMHead(s.hidden, s.vocab, tile_k=tile_k, tile_n=tile_n)
    head_dense = fill(head, head_w)
    comp["head"], ref["head"] = head, (lambda x, w=head_dense: torch.matmul(x, w.t()))
    same["head"] = lambda x, w=head_dense: ci.plain_linear_transposed_same_order(x, w, tile_k=tile_k, tile_n=tile_n)
    return comp, ref, same, sizes


def run(n_layers=32, n_prompt=128, n_new=256, tile_k=1024, tile_n=32, gen="cpu"):
    import comp_inference_amd as ci  # noqa: F401

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    log(f"building the {n_layers}-layer decoder (generator: {gen}) ...")
    comp, ref, same, sizes = build(n_layers, dev, tile_k, tile_n, gen)
    prompt = torch.randint(0, Shape.vocab, (n_prompt,), generator=torch.Generator("cpu").manual_seed(6)).to(dev)
    max_len = n_prompt + n_new + 1
    res = {}
    with torch.no_grad():
        for name, ops, graph in (("reference_bf16", ref, False), ("reference_bf16_graph", ref, True),
                                 ("compressed_eager", comp, False), ("compressed_graph", comp, True),
                                 ("decompressed_same_order", same, False)):
            log(f"decoding: {name} ...")
            dec = Decoder(ops, n_layers, max_len, dev)
            ids, sec = generate(dec, prompt, n_new, graph)
            res[name] = (ids, sec)
            del dec
    # the decoder-checkpoint indexes the compressed modules built for themselves on first use
    index_bytes = 0
    for mods in ([comp["embed"], comp["head"]], comp["qkv"], comp["o"], comp["gate_up"], comp["down"]):
        for m in mods:
            ck = getattr(m, "_ckpt_cache", None)
            if ck is not None and ck[1] is not None:
                index_bytes += ck[1].numel() * 8
    base = res["reference_bf16"][0]
    with torch.no_grad():
        log("teacher-forced comparison ...")
        lr = teacher_forced(Decoder(ref, n_layers, max_len, dev), prompt, base)
        lc = teacher_forced(Decoder(comp, n_layers, max_len, dev), prompt, base)
        ls = teacher_forced(Decoder(same, n_layers, max_len, dev), prompt, base)
    logits_bit_identical = bool(torch.equal(lc, ls))
    del ls
    forced_same = int((lr.argmax(-1) == lc.argmax(-1)).sum())
    logit_err = float((lr - lc).abs().max())
    top2 = lr.topk(2, dim=-1).values
    min_gap = float((top2[:, 0] - top2[:, 1]).min())

    def agree(ids):
        n = 0
        for a, b in zip(ids, base):
            if a != b:
                break
            n += 1
        return n

    return {
        "model": f"Llama-3-8B shape, {n_layers} layers, random init seed 5 ({gen} generator), tile {tile_k}x{tile_n}",
        "prompt_tokens": n_prompt, "new_tokens": n_new,
        "weight_bytes_compressed": sizes["compressed"], "weight_bytes_bf16": sizes["bf16"],
        "checkpoint_index_bytes": int(index_bytes),
        "tok_per_s_compressed_graph": round(n_new / res["compressed_graph"][1], 2),
        "tok_per_s_compressed_eager": round(n_new / res["compressed_eager"][1], 2),
        "tok_per_s_reference_bf16_graph": round(n_new / res["reference_bf16_graph"][1], 2),
        "tok_per_s_reference_bf16_eager": round(n_new / res["reference_bf16"][1], 2),
        # the run on decompressed weights in the fused kernels' contraction order: equal ids and equal
        # logit bits mean every weight bit is reconstructed and nothing else differs
        "ids_equal_to_decompressed_same_order_run": res["compressed_eager"][0] == res["decompressed_same_order"][0],
        "graph_ids_equal_to_decompressed_same_order_run":
            res["compressed_graph"][0] == res["decompressed_same_order"][0],
        "teacher_forced_logits_bit_identical_to_same_order_run": logits_bit_identical,
        # the run on decompressed weights through hipBLASLt sums in another order
        "ids_equal_to_reference": res["compressed_eager"][0] == base,
        "ids_matching_prefix": agree(res["compressed_eager"][0]),
        "teacher_forced_top1_agreement": f"{forced_same}/{n_new}",
        "teacher_forced_max_abs_logit_diff": round(logit_err, 5),
        "reference_smallest_top1_top2_logit_gap": round(min_gap, 6),
        "graph_ids_equal_eager_ids": res["compressed_graph"][0] == res["compressed_eager"][0],
        "reference_graph_ids_equal_eager_ids": res["reference_bf16_graph"][0] == base,
        "first_ids": res["compressed_eager"][0][:8],
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--prompt", type=int, default=128)
    ap.add_argument("--new", type=int, default=256)
    ap.add_argument("--tile-k", type=int, default=1024)
    ap.add_argument("--gen", choices=("cpu", "cuda"), default="cpu")
    a = ap.parse_args()
    if not torch.cuda.is_available():
        print("bench_model.py needs a GPU (gfx950)", file=sys.stderr)
        return 2
    print(json.dumps(run(a.layers, a.prompt, a.new, a.tile_k, 32, a.gen)))
    return 0


if __name__ == "__main__":
    sys.exit(main())
