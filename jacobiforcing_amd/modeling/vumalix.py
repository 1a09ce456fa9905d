"""Vumalix: a decoder with a float residual stream in which the norms sit on the sublayers' OUTPUTS (x += g * unit_rms(sublayer(x)),
g one number per norm), every mixer reads the stream through a short causal convolution over time, and a layer may borrow another
layer's weights while keeping a cache of its own.

* mixer ``attention``: differential attention.  Every head has two score maps over the same values (grouped-query layout); query
  and key are RMS-normalised per head and map; positions enter only through a query temperature that grows with the logarithm of
  the position's block number; the maps' outputs are combined as a1 - lambda * a2, brought to unit RMS per head and scaled.
* mixer ``latent_attention``: queries and keys/values go through low-rank latents.  The pool keeps, per token, the normalised
  key/value latent and one rotary key part shared by the heads; the query is multiplied by the key up-projection instead of the
  cached latents, so attention runs over the pool with a single key/value head and the value up-projection follows it.  Sliding
  window, sigmoid output gate.
* feed-forward: down(act(up x)) with a polynomial activation whose three powers are each brought to unit RMS.

The forward runs one ragged batch (``layer_ops.RaggedBatch``) over ``engine.state_cache.PagedStateCache``: pages for the pools, a
slot per request for the convolutions' last inputs.  Dense products are torch's (hipBLASLt / rocBLAS); everything else is a launch
of ``libjf_layers.so``.  With float32 weights every product is a true 32-bit one."""
from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Dict, List, Optional

import torch
import torch.nn.functional as F

from .. import layer_ops as LO
from ..engine.state_cache import PagedStateCache, RunSpec

MIXERS = ("attention", "latent_attention")


@dataclass
class VumalixConfig:
    vocab_size: int
    hidden_size: int
    layers: List[Dict[str, Any]]
    norm_eps: float = 1e-6
    conv_taps: int = 1
    max_position_embeddings: int = 1 << 20          # the design has no limit of its own: the engine's max_model_len decides
    eos_token_id: int = -1
    pad_token_id: int = 0
    family: str = "ragged"

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    def weights_layer(self, i: int) -> int:
        """The layer whose tensors layer i uses (itself unless it borrows; a borrowed layer that borrows in turn is followed)."""
        seen = set()
        while self.layers[i].get("weights_of") is not None and i not in seen:
            seen.add(i)
            i = int(self.layers[i]["weights_of"])
        return i

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "VumalixConfig":
        layers = d["layers"]
        taps = int((d.get("canon") or {}).get("taps", 1))
        if not 1 <= taps <= 16:
            raise ValueError(f"canon.taps {taps} is outside 1..16")
        for i, L in enumerate(layers):
            if L["type"] not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer {L['type']!r}")
            if L.get("mlp") is not None and L["mlp"].get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward {L['mlp'].get('kind')!r}")
            j = L.get("weights_of")
            if j is not None:
                j, hops = int(j), 0
                while 0 <= j < len(layers) and layers[j].get("weights_of") is not None and hops < len(layers):
                    j, hops = int(layers[j]["weights_of"]), hops + 1
                if not 0 <= j < len(layers) or layers[j].get("weights_of") is not None or layers[j]["type"] != L["type"]:
                    raise ValueError(f"layer {i}: weights_of must lead to a layer of the same type that owns its tensors")
            m = L["mixer"]
            if L["type"] == "attention" and int(m["heads"]) % int(m["kv_heads"]):
                raise ValueError(f"layer {i}: {m['heads']} heads over {m['kv_heads']} key/value heads")
            if L["type"] == "latent_attention":
                rot = m.get("rot") or {}
                dims = int(rot.get("dims", 0))
                if dims % 2 or dims > int(m["rot_dim"]):
                    raise ValueError(f"layer {i}: rot.dims {dims} must be even and at most rot_dim {m['rot_dim']}")
        return cls(vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), layers=layers, norm_eps=float(d["norm"]["eps"]), conv_taps=taps,
                   eos_token_id=int(d.get("eos_token_id", -1)), pad_token_id=int(d.get("pad_token_id", 0)))

    @classmethod
    def from_json(cls, path) -> "VumalixConfig":
        return cls.from_dict(json.loads(Path(path).read_text()))


class VumalixWeights:
    """Tensors by their checkpoint names (``embed``, ``l<i>.norm1``, ``l<i>.canon1``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``,
    ``head``), regrouped per layer for the forward: a mixer's input projections stacked into one matrix, the latent
    up-projections per head ([H, D, R] for keys, [H, R, Dv] for values), single-number norm weights and the activation's
    coefficients in float.  A layer that borrows weights shares the owner's entry."""

    def __init__(self, cfg: VumalixConfig, tensors: Dict[str, torch.Tensor], device, dtype=torch.bfloat16):
        dev = torch.device(device)
        act = lambda k: tensors[k].to(device=dev, dtype=dtype).contiguous()
        f32 = lambda k: tensors[k].to(device=dev, dtype=torch.float32).reshape(-1).contiguous()
        self.device, self.dtype = dev, dtype
        W = cfg.hidden_size
        self.embed, self.head = act("embed"), act("head")
        # the model's last norm has one weight too; the shared norm launch wants one per column
        self.final_norm = tensors["final.norm"].to(device=dev, dtype=dtype).reshape(-1)[:1].expand(W).contiguous()
        if tuple(self.embed.shape) != (cfg.vocab_size, W):
            raise ValueError(f"embed is {tuple(self.embed.shape)}, config says {(cfg.vocab_size, W)}")
        self.layers: List[Optional[dict]] = [None] * len(cfg.layers)
        for i, L in enumerate(cfg.layers):
            if cfg.weights_layer(i) != i:
                continue
            p, m = f"l{i}.", L["mixer"]
            w = dict(type=L["type"], norm1=f32(p + "norm1"), canon=act(p + "canon1"), w_o=act(p + "mix.o"))
            if tuple(w["canon"].shape) != (W, cfg.conv_taps):
                raise ValueError(f"layer {i}: canon1 is {tuple(w['canon'].shape)}, config says {(W, cfg.conv_taps)}")
            if L["type"] == "attention":
                H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
                w.update(w_in=torch.cat([act(p + "mix.q"), act(p + "mix.k"), act(p + "mix.v")], 0), cols=(0, 2 * H * D, 2 * H * D + 2 * G * D),
                         q_norm=act(p + "mix.q.norm"), k_norm=act(p + "mix.k.norm"))
                want = 2 * H * D + 2 * G * D + G * Dv
                t = {k: tensors[p + "mix." + k].float() for k in ("lq1", "lk1", "lq2", "lk2")}
                w["lam"] = float(torch.exp((t["lq1"] * t["lk1"]).sum()) - torch.exp((t["lq2"] * t["lk2"]).sum()) + torch.tensor(float(m["diff"])))
            else:
                H, D, rd, Dv, R, Rq = (int(m[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"))
                w.update(w_in=torch.cat([act(p + "mix.dq"), act(p + "mix.dkv"), act(p + "mix.g")], 0), cols=(0, Rq, Rq + R + rd),
                         dq_norm=act(p + "mix.dq.norm"), dkv_norm=act(p + "mix.dkv.norm"), w_uq=act(p + "mix.uq"),
                         w_uk=act(p + "mix.uk").view(H, D, R).contiguous(), w_uv=act(p + "mix.uv").view(H, Dv, R).transpose(1, 2).contiguous())
                want = Rq + R + rd + H * Dv
                if tuple(w["w_uq"].shape) != (H * (D + rd), Rq):
                    raise ValueError(f"layer {i}: uq is {tuple(w['w_uq'].shape)}, the config's sizes give {(H * (D + rd), Rq)}")
            if w["w_in"].shape[0] != want:
                raise ValueError(f"layer {i}: projections have {w['w_in'].shape[0]} rows, the config's sizes give {want}")
            if L.get("mlp") is not None:
                w.update(norm2=f32(p + "norm2"), w_up=act(p + "mlp.up"), w_down=act(p + "mlp.down"), act=f32(p + "mlp.act"))
                if w["w_up"].shape[0] != int(L["mlp"]["ff"]):
                    raise ValueError(f"layer {i}: up is {tuple(w['w_up'].shape)}, config says ff {L['mlp']['ff']}")
            self.layers[i] = w
        for i in range(len(cfg.layers)):
            self.layers[i] = self.layers[cfg.weights_layer(i)]

    @classmethod
    def from_safetensors(cls, cfg: VumalixConfig, model_dir, device, dtype=torch.bfloat16) -> "VumalixWeights":
        from safetensors import safe_open
        files = sorted(Path(model_dir).glob("*.safetensors"))
        if not files:
            raise FileNotFoundError(f"no *.safetensors under {model_dir}")
        tensors = {}
        for f in files:
            with safe_open(str(f), "pt", "cpu") as sf:
                for k in sf.keys():
                    tensors[k] = sf.get_tensor(k)
        return cls(cfg, tensors, device, dtype)

    @classmethod
    def random(cls, cfg: VumalixConfig, device, dtype=torch.bfloat16, seed: int = 0) -> "VumalixWeights":
        return cls(cfg, random_tensors(cfg, seed), device, dtype)


def random_tensors(cfg: VumalixConfig, seed: int = 0) -> Dict[str, torch.Tensor]:
    """Random tensors under the checkpoint's names (benchmarks and tests; bf16-representable float32 values)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg.hidden_size
    rnd = lambda *s, std=1.0: (torch.randn(*s, generator=g) * std).to(torch.bfloat16).float()
    lin = lambda o, i: rnd(o, i, std=i ** -0.5)
    one = lambda *s: (1 + torch.randn(*s, generator=g) * 0.1).to(torch.bfloat16).float()
    t = {"embed": rnd(cfg.vocab_size, W), "final.norm": one(()), "head": lin(cfg.vocab_size, W)}
    for i, L in enumerate(cfg.layers):
        if cfg.weights_layer(i) != i:
            continue
        p, m = f"l{i}.", L["mixer"]
        t[p + "norm1"] = one(()) * 0.5
        t[p + "canon1"] = rnd(W, cfg.conv_taps, std=0.3)
        if L["type"] == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            t.update({p + "mix.q": lin(2 * H * D, W), p + "mix.k": lin(2 * G * D, W), p + "mix.v": lin(G * Dv, W), p + "mix.o": lin(W, H * Dv),
                      p + "mix.q.norm": one(D), p + "mix.k.norm": one(D)})
            for k in ("lq1", "lk1", "lq2", "lk2"):
                t[p + "mix." + k] = rnd(D, std=0.1)
        else:
            H, D, rd, Dv, R, Rq = (m[k] for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"))
            t.update({p + "mix.dq": lin(Rq, W), p + "mix.dq.norm": one(Rq), p + "mix.uq": lin(H * (D + rd), Rq), p + "mix.dkv": lin(R + rd, W),
                      p + "mix.dkv.norm": one(R), p + "mix.uk": lin(H * D, R), p + "mix.uv": lin(H * Dv, R), p + "mix.g": lin(H * Dv, W),
                      p + "mix.o": lin(W, H * Dv)})
        if L.get("mlp") is not None:
            ff = L["mlp"]["ff"]
            t.update({p + "norm2": one(()) * 0.5, p + "mlp.up": lin(ff, W), p + "mlp.down": lin(W, ff), p + "mlp.act": rnd(4, std=0.5)})
    return t


class VumalixModel:
    def __init__(self, cfg: VumalixConfig, weights: VumalixWeights, max_positions: int = 8192):
        self.cfg, self.w = cfg, weights
        self.device, self.dtype = weights.device, weights.dtype
        self._angles: Dict[tuple, tuple] = {}
        self.max_positions = 0
        self.reserve_positions(max_positions)

    # ---- what the cache must hold, one entry per layer (a layer that borrows weights has pages and a slot entry of its own) --------
    def cache_specs(self) -> List[RunSpec]:
        tail = (self.cfg.conv_taps - 1, self.cfg.hidden_size)
        specs = []
        for L in self.cfg.layers:
            m = L["mixer"]
            if L["type"] == "attention":        # both score maps' keys side by side; one set of values
                specs.append(RunSpec("kv", k_width=2 * m["kv_heads"] * m["dim"], v_width=m["kv_heads"] * m["vdim"], tail_shape=tail))
            else:                               # the latent and the shared rotary key; values are read out of the same rows
                specs.append(RunSpec("kv", k_width=m["kv_rank"] + m["rot_dim"], v_width=0, tail_shape=tail))
        return specs

    def new_cache(self, num_pages: int, page_size: int, num_slots: int) -> PagedStateCache:
        return PagedStateCache(self.cache_specs(), num_pages, page_size, num_slots, self.device, self.dtype)

    # ---- rotation angles for every position the engine can reach, in float ---------------------------------------------------------
    def reserve_positions(self, n: int) -> None:
        if n <= self.max_positions:
            return
        self.max_positions = int(n)
        self._angles.clear()
        for L in self.cfg.layers:
            rot = L["mixer"].get("rot") or {}
            dims, base = int(rot.get("dims", 0)), float(rot.get("base", 10000.0))
            if L["type"] == "latent_attention" and dims and (dims, base) not in self._angles:
                f = torch.tensor([base ** (-2.0 * k / dims) for k in range(dims // 2)], dtype=torch.float32, device=self.device)
                a = torch.arange(n, dtype=torch.float32, device=self.device).view(n, 1) * f.view(1, -1)
                self._angles[(dims, base)] = (a.cos().contiguous(), a.sin().contiguous())

    # ---- mixers ------------------------------------------------------------------------------------------------------------------
    def _attention(self, li: int, h: torch.Tensor, batch: LO.RaggedBatch, cache: PagedStateCache) -> torch.Tensor:
        m, w, eps = self.cfg.layers[li]["mixer"], self.w.layers[li], self.cfg.norm_eps
        H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
        qt = m.get("q_temp") or {}
        proj = F.linear(h, w["w_in"])
        kp, vp, scale = cache.k[li], cache.v[li], float(m["scale"])
        window = int((m.get("mask") or {}).get("size", 0))                                          # none in the design: plain causal
        sweep = LO.attn_sweep_tile_rows(self.dtype, 2 * H, 2 * G, D, Dv, kp, vp, G) > 0
        apart = 2 * H > LO.ATTN_MAX_HEADS_ONE_LAUNCH and not sweep
        q = LO.head_norm_append(proj, w["cols"], H, G, 2, D, Dv, w["q_norm"], w["k_norm"], eps, float(qt.get("coef", 0.0)), int(qt.get("every", 1)),
                                batch, cache.k[li], cache.v[li], maps_apart=apart)
        if sweep:       # bfloat16: both maps of all heads in one one-sweep launch (2G groups of H/G heads, G value heads)
            a = LO.attn_sweep(q, kp, vp, batch, 2 * H, 2 * G, D, Dv, scale, window, value_heads=G, float_out=True)
            a1, a2 = a[:, :H * Dv], a[:, H * Dv:]
        elif not apart:   # one launch for both maps: 2H query heads over 2G key heads and G value heads, plain causal, float outputs
            a = LO.attn_window(q, None, kp, vp, batch, 2 * H, 2 * G, D, Dv, scale, window, 0, None, None, None, value_heads=G, float_out=True)
            a1, a2 = a[:, :H * Dv], a[:, H * Dv:]
        else:           # more heads than one workgroup takes: a launch per map over its own columns of the key rows
            a1, a2 = (LO.attn_window(q[mp], None, kp[:, mp * G * D:(mp + 1) * G * D], vp, batch, H, G, D, Dv, scale, window, 0, None, None, None,
                                     float_out=True) for mp in range(2))
        return LO.diff_combine(a1, a2, H, Dv, w["lam"], eps, 1.0 - float(m["diff"]), self.dtype)

    def _latent_attention(self, li: int, h: torch.Tensor, batch: LO.RaggedBatch, cache: PagedStateCache) -> torch.Tensor:
        m, w, eps = self.cfg.layers[li]["mixer"], self.w.layers[li], self.cfg.norm_eps
        H, D, rd, Dv, R, Rq = (int(m[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"))
        rot = m.get("rot") or {}
        dims = int(rot.get("dims", 0))
        cos, sin = self._angles[(dims, float(rot.get("base", 10000.0)))] if dims else (None, None)
        n = h.shape[0]
        pool = cache.k[li]
        proj = F.linear(h, w["w_in"])
        cq = LO.latent_prep(proj, w["cols"][0], Rq, w["cols"][1], R, rd, dims, w["dq_norm"], w["dkv_norm"], eps, batch, cos, sin, pool)
        q = F.linear(cq, w["w_uq"])
        qa = torch.bmm(q.view(n, H, D + rd)[:, :, :D].transpose(0, 1), w["w_uk"])                    # [H, N, R]: query . (W_uk c) = (W_uk^T query) . c
        qf = LO.latent_q_pack(qa, q, H, D, R, rd, dims, batch, cos, sin)
        window, scale = int((m.get("mask") or {}).get("size", 0)), float(m["scale"])
        step = LO.ATTN_MAX_VALUE_WIDTH
        if LO.attn_sweep_tile_rows(self.dtype, H, 1, R + rd, R, pool, pool[:, :R]):                 # bfloat16, latents in multiples of 32 up to 512
            o = LO.attn_sweep(qf, pool, pool[:, :R], batch, H, 1, R + rd, R, scale, window)
            ov = torch.bmm(o.view(n, H, R).transpose(0, 1), w["w_uv"])
        elif R <= step or self.dtype != torch.bfloat16:
            o = LO.attn_window(qf, None, pool, pool[:, :R], batch, H, 1, R + rd, R, scale, window, 0, None, None, None)
            ov = torch.bmm(o.view(n, H, R).transpose(0, 1), w["w_uv"])                               # [H, N, Dv]
        else:           # a latent wider than the matrix-core kernel's value tile: a launch per column range of the latent
            ov = None
            for c0 in range(0, R, step):
                c1 = min(R, c0 + step)
                o = LO.attn_window(qf, None, pool, pool[:, c0:c1], batch, H, 1, R + rd, c1 - c0, scale, window, 0, None, None, None)
                o = o.view(n, H, c1 - c0).transpose(0, 1)
                ov = torch.bmm(o, w["w_uv"][:, c0:c1]) if ov is None else torch.baddbmm(ov, o, w["w_uv"][:, c0:c1])
        return LO.heads_gate(ov, proj[:, w["cols"][2]:w["cols"][2] + H * Dv])

    # ---- one step ----------------------------------------------------------------------------------------------------------------
    @torch.inference_mode()
    def forward(self, ids: torch.Tensor, batch: LO.RaggedBatch, cache: PagedStateCache, logit_rows: Optional[torch.Tensor] = None,
                trace: Optional[list] = None) -> torch.Tensor:
        """ids int64 [N] (the batch's rows).  Returns float logits [N, vocab], or of the rows in ``logit_rows``.  ``trace``, when a
        list, receives the residual stream after every layer (debugging and tests)."""
        cfg, w, eps, dt = self.cfg, self.w, self.cfg.norm_eps, self.dtype
        if batch.max_pos > self.max_positions:
            raise ValueError(f"position {batch.max_pos - 1} is beyond the {self.max_positions} positions the tables were reserved for")
        x, _ = LO.embed_scale(w.embed, ids, 1.0, False)
        for li, L in enumerate(cfg.layers):
            lw = w.layers[li]
            h = LO.causal_conv(x, lw["canon"], batch, cache.tail[li])
            a = self._attention(li, h, batch, cache) if L["type"] == "attention" else self._latent_attention(li, h, batch, cache)
            y = F.linear(a, lw["w_o"])
            if L.get("mlp") is not None:
                h2 = LO.norm_add(x, y, lw["norm1"], eps, dt)
                act = LO.polynorm(F.linear(h2, lw["w_up"]), lw["act"], eps)
                LO.norm_add(x, F.linear(act, lw["w_down"]), lw["norm2"], eps, None)
            else:
                LO.norm_add(x, y, lw["norm1"], eps, None)
            if trace is not None:
                trace.append(x.clone())
        hf = LO.add_rmsnorm(x, None, None, w.final_norm, eps, dt)
        if logit_rows is not None:
            hf = hf.index_select(0, logit_rows)
        return F.linear(hf, w.head).float()


def load_model_directory(model_dir, device, dtype=torch.bfloat16, max_positions: int = 8192):
    cfg = VumalixConfig.from_json(Path(model_dir) / "config.json")
    return cfg, VumalixModel(cfg, VumalixWeights.from_safetensors(cfg, model_dir, device, dtype), max_positions)


def random_model(cfg: VumalixConfig, device, dtype=torch.bfloat16, max_positions: int = 8192, seed: int = 0) -> VumalixModel:
    return VumalixModel(cfg, VumalixWeights.random(cfg, device, dtype, seed), max_positions)
