#!/usr/bin/env python3
"""Prefill and decode throughput of a ragged model family (Lokizen) at sizes that resemble a real model's layers, beside the
package's Qwen2 forward at equal width, depth, head sizes and active feed-forward width — random weights, synthetic tokens.

    python -m jacobiforcing_amd.drivers.ragged_bench [--sizes small,medium] [--kernels]
    python bench.py --design lokizen            (the same, as one JSON line)

Per size: prefill = whole prompts in one step (tokens / s), decode = one token for each of ``--decode-batch`` requests at a
context of ``--context`` tokens (tokens / s).  ``--kernels`` adds each layer kernel alone at the size's shapes with its
algorithmic bytes and flops and the fraction of the chip's roofline (8 TB/s, 2.5 PFLOP/s bf16 matrix / 157 TFLOP/s float
vector) that its time amounts to, next to the like kernel of the Qwen2 forward (scaled-dot-product attention, the SwiGLU
launch, F.rms_norm)."""
from __future__ import annotations

import argparse
import json
import time

import torch
import torch.nn.functional as F

HBM_BPS, MATRIX_FLOPS, VECTOR_FLOPS = 8.0e12, 2.5e15, 157e12

SIZES = {
    # width, layers (alternating retention / attention), heads, kv_heads, dim, experts, top, ff, window, vocab
    "small": dict(width=1024, layers=4, heads=8, kv=2, dim=128, experts=16, top=4, ff=512, window=1024, vocab=32000),
    "medium": dict(width=2048, layers=8, heads=16, kv=4, dim=128, experts=32, top=4, ff=1024, window=2048, vocab=32000),
}


def lokizen_config(s):
    from ..modeling.lokizen import LokizenConfig
    H, D = s["heads"], s["dim"]
    moe = {"kind": "moe", "expert": {"ff": s["ff"]}, "router": {"experts": s["experts"], "top": s["top"], "scale": 1.0}}
    ret = {"type": "retention", "mlp": moe, "mixer": {"heads": H, "dim": D, "vdim": D, "rot": {"dims": D, "base": 1e6},
                                                       "decay": [1 - 2.0 ** (-5 - 3 * h / H) for h in range(H)]}}
    att = {"type": "attention", "mlp": moe, "mixer": {"heads": H, "kv_heads": s["kv"], "dim": D, "vdim": D, "scale": D ** -0.5, "bias_max": 4096,
                                                       "mask": {"size": s["window"], "keep_first": 4}}}
    return LokizenConfig.from_dict({"architecture": "Lokizen", "vocab": s["vocab"], "width": s["width"], "norm": {"eps": 1e-5},
                                    "embedding": {"scale": 1.0}, "layers": [ret if i % 2 == 0 else att for i in range(s["layers"])]})


def qwen2_config(s):
    from ..modeling.qwen2 import Qwen2Config
    return Qwen2Config(vocab_size=s["vocab"], hidden_size=s["width"], intermediate_size=s["top"] * s["ff"], num_hidden_layers=s["layers"],
                       num_attention_heads=s["heads"], num_key_value_heads=s["kv"], head_dim=s["dim"], max_position_embeddings=1 << 16,
                       eos_token_id=s["vocab"] - 1, pad_token_id=s["vocab"] - 2)


def timed(fn, warmup=2, iters=5):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / iters


def bench_lokizen(s, prompts, prompt_len, decode_batch, context, dtype=torch.bfloat16):
    from .. import layer_ops as LO
    from ..modeling.lokizen import random_model
    dev = "cuda"
    model = random_model(lokizen_config(s), dev, dtype, max_positions=max(prompt_len, context) + 64)
    page = 64
    per = -(-(max(prompt_len, context) + 1) // page)
    slots = max(prompts, decode_batch)
    cache = model.new_cache(slots * per, page, slots)
    tables = [list(range(b * per, (b + 1) * per)) for b in range(slots)]
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, s["vocab"], (prompts * prompt_len,), generator=g).to(dev)
    pre = LO.RaggedBatch.build([prompt_len] * prompts, [0] * prompts, list(range(prompts)), tables[:prompts], page, dev)
    last = torch.arange(prompts, device=dev) * prompt_len + prompt_len - 1
    t_pre = timed(lambda: model.forward(ids, pre, cache, last))
    # decode at `context`: the pool holds whatever the prompts left (random weights: the timing does not depend on the values)
    dec = LO.RaggedBatch.build([1] * decode_batch, [context] * decode_batch, list(range(decode_batch)), tables[:decode_batch], page, dev)
    dids = ids[:decode_batch].contiguous()
    t_dec = timed(lambda: model.forward(dids, dec, cache, None), warmup=3, iters=20)
    return {"prefill_tokens_per_s": prompts * prompt_len / t_pre, "prefill_ms": 1e3 * t_pre, "decode_tokens_per_s": decode_batch / t_dec,
            "decode_ms": 1e3 * t_dec}


def bench_qwen2(s, prompts, prompt_len, decode_batch, context, dtype=torch.bfloat16):
    from ..modeling.qwen2 import Qwen2Model, Qwen2Weights, StaticKVCache
    dev = torch.device("cuda")
    cfg = qwen2_config(s)
    model = Qwen2Model(cfg, Qwen2Weights(cfg, dev, dtype=dtype))
    g = torch.Generator().manual_seed(0)

    def run(R, T, start, last_only):
        cache = StaticKVCache(cfg, R, start + T + 8, 0, 1, dev, dtype=dtype)          # row r of the batch is cache row r: attended in place
        ids = torch.randint(0, s["vocab"], (R, T), generator=g).to(dev)
        st = torch.full((R,), start, dtype=torch.int32, device=dev)
        pos = st.view(R, 1) + torch.arange(T, dtype=torch.int32, device=dev).view(1, T)
        rp = torch.arange(R, dtype=torch.int32, device=dev)
        idx = (torch.arange(R, dtype=torch.int32, device=dev) * T + T - 1) if last_only else None
        return lambda: model.forward(ids, pos, cache, row_prompt=rp, row_cand=rp * 0 - 1, row_len=st * 0 + T, kv_len_rows=st, any_candidates=False,
                                     s_cur=start + T, logit_index=idx, rows_in_place=True)

    t_pre = timed(run(prompts, prompt_len, 0, True))
    t_dec = timed(run(decode_batch, 1, context, False), warmup=3, iters=20)
    return {"prefill_tokens_per_s": prompts * prompt_len / t_pre, "prefill_ms": 1e3 * t_pre, "decode_tokens_per_s": decode_batch / t_dec,
            "decode_ms": 1e3 * t_dec}


def kernel_table(s, prompts, prompt_len, decode_batch, context, dtype=torch.bfloat16):
    """Each layer kernel alone, prefill shape and decode shape: microseconds, algorithmic bytes / flops, fraction of the roofline
    (the larger of bytes / 8 TB/s and flops / peak, over the time)."""
    from .. import layer_ops as LO
    from .. import ops
    dev = "cuda"
    H, G, D, W, E, top, ff, win = s["heads"], s["kv"], s["dim"], s["width"], s["experts"], s["top"], s["ff"], s["window"]
    page, es = 64, 2
    per = -(-(max(prompt_len, context) + 1) // page)
    slots = max(prompts, decode_batch)
    tables = [list(range(b * per, (b + 1) * per)) for b in range(slots)]
    g = torch.Generator().manual_seed(0)
    rnd = lambda *sh: torch.randn(*sh, generator=g).to(dev).to(dtype)
    kc, vc = rnd(slots * per * page, G * D), rnd(slots * per * page, G * D)
    state = torch.zeros((slots, H, D, D), device=dev)
    decay = torch.full((H,), 0.99, device=dev)
    a = torch.arange(max(prompt_len, context) + 8, dtype=torch.float32, device=dev).view(-1, 1) * torch.rand(D // 2, device=dev).view(1, -1)
    cos, sin = a.cos().contiguous(), a.sin().contiguous()
    rel, talk = torch.randn(16, H, device=dev), torch.eye(H, device=dev)
    from ..modeling.lokizen import distance_bucket_table
    lut = torch.from_numpy(distance_bucket_table(16, 4096, max(prompt_len, context) + 8)).to(dev)
    rel, lut = rel[lut.long()].contiguous(), None                       # the bias laid out by distance, as the model passes it
    w_up, w_down = rnd(E, ff, W) * 0.02, rnd(E, W, ff) * 0.02
    out = {}

    def row(name, secs, nbytes, flops, peak):
        bound = max(nbytes / HBM_BPS, flops / peak)
        out[name] = {"us": round(1e6 * secs, 1), "MB": round(nbytes / 1e6, 2), "GFLOP": round(flops / 1e9, 2), "roofline_fraction": round(bound / secs, 4)}

    for phase, B, T, start in (("prefill", prompts, prompt_len, 0), ("decode", decode_batch, 1, context)):
        n = B * T
        batch = LO.RaggedBatch.build([T] * B, [start] * B, list(range(B)), tables[:B], page, dev)
        x, y, wn = torch.randn(n, W, device=dev), rnd(n, W), rnd(W)
        row(f"{phase}.add_rmsnorm", timed(lambda: LO.add_rmsnorm(x, y, None, wn, 1e-5, dtype)), n * W * (4 + 4 + es + es), 4.0 * n * W, VECTOR_FLOPS)
        q, gate = rnd(n, H * D), rnd(n, H * D)
        keys = sum(min(start + t + 1, win + 4) for t in range(T)) * B                       # visible (query, key) pairs per head
        kv_bytes = B * min(start + T, win + T) * 2 * G * D * es                              # every needed key / value row once
        t_att = timed(lambda: LO.attn_window(q, gate, kc, vc, batch, H, G, D, D, D ** -0.5, win, 4, rel, lut, talk))
        row(f"{phase}.attn_window", t_att, kv_bytes + 3 * n * H * D * es, 4.0 * keys * H * D, MATRIX_FLOPS)
        proj = rnd(n, 4 * H * D)
        t_ret = timed(lambda: LO.retention(proj, (0, H * D, 2 * H * D, 3 * H * D), batch, H, D, D, D, cos, sin, decay, 1e-5, state))
        row(f"{phase}.retention", t_ret, n * 5 * H * D * es + 2 * B * H * D * D * 4, 4.0 * n * H * D * D, VECTOR_FLOPS)
        h, z = rnd(n, W), torch.randn(n, E, device=dev)
        t_moe = timed(lambda: LO.moe_experts(h, z, None, top, 1.0, w_up, w_down))
        used = min(E, n * top)
        row(f"{phase}.moe_experts", t_moe, used * 2 * ff * W * es + n * W * es + n * top * W * 4, 4.0 * n * top * ff * W, MATRIX_FLOPS)
        # the like kernels of the Qwen2 forward at the same shapes
        S = start + T
        qh = rnd(B, G, (H // G) * T, D)
        Kf, Vf = rnd(B, G, S, D), rnd(B, G, S, D)
        bias = torch.zeros((B, 1, (H // G) * T, (S + 15) // 16 * 16), dtype=dtype, device=dev)[..., :S]
        t_sdpa = timed(lambda: F.scaled_dot_product_attention(qh, Kf, Vf, attn_mask=bias))
        pairs = B * sum(start + t + 1 for t in range(T))
        row(f"{phase}.qwen2.sdpa", t_sdpa, 2 * B * S * G * D * es + 2 * n * H * D * es, 4.0 * pairs * H * D, MATRIX_FLOPS)
        gu = rnd(n, 2 * top * ff)
        row(f"{phase}.qwen2.swiglu", timed(lambda: ops.swiglu(gu)), 3 * n * top * ff * es, 4.0 * n * top * ff, VECTOR_FLOPS)
        xb = rnd(n, W)
        row(f"{phase}.qwen2.rms_norm", timed(lambda: F.rms_norm(xb, (W,), wn, 1e-5)), 2 * n * W * es, 4.0 * n * W, VECTOR_FLOPS)
        wgu, wd = rnd(2 * top * ff, W), rnd(W, top * ff)
        t_mlp = timed(lambda: F.linear(ops.swiglu(F.linear(xb, wgu)), wd))
        row(f"{phase}.qwen2.mlp_gemms", t_mlp, 3 * top * ff * W * es + 2 * n * W * es, 6.0 * n * top * ff * W, MATRIX_FLOPS)
    return out


def run(sizes=("small", "medium"), prompts=4, prompt_len=2048, decode_batch=32, context=2048, kernels=True):
    res = {"bench": "ragged_family", "design": "Lokizen", "closest": "Qwen2", "dtype": "bf16", "data": "synthetic", "prompts": prompts,
           "prompt_len": prompt_len, "decode_batch": decode_batch, "context": context, "sizes": {}}
    for name in sizes:
        s = SIZES[name]
        entry = {"shape": s, "lokizen": bench_lokizen(s, prompts, prompt_len, decode_batch, context)}
        torch.cuda.empty_cache()
        entry["qwen2"] = bench_qwen2(s, prompts, prompt_len, decode_batch, context)
        torch.cuda.empty_cache()
        if kernels:
            entry["kernels"] = kernel_table(s, prompts, prompt_len, decode_batch, context)
            torch.cuda.empty_cache()
        res["sizes"][name] = entry
    return res


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--sizes", default="small,medium")
    ap.add_argument("--prompts", type=int, default=4)
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--decode-batch", type=int, default=32)
    ap.add_argument("--context", type=int, default=2048)
    ap.add_argument("--no-kernels", action="store_true")
    a = ap.parse_args(argv)
    print(json.dumps(run(tuple(a.sizes.split(",")), a.prompts, a.prompt_len, a.decode_batch, a.context, not a.no_kernels)), flush=True)


if __name__ == "__main__":
    main()
