"""Lokizen: a decoder with a float residual stream whose layers pair one of two token mixers with routed experts, and which may
run a span of its layers several times with the same weights.

* mixer ``attention``: grouped-query attention without rotation; query and key are RMS-normalised over the WHOLE projection;
  positions enter through a sliding window that keeps the sequence's first tokens and through a learned bias indexed by a
  bucketed distance; after the softmax the heads' weights are mixed by a learned [H, H] matrix; a sigmoid gate multiplies the
  heads' outputs before the output projection.
* mixer ``retention``: S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head, rotary positions on q / k, unit RMS per head,
  a silu gate.  The state is float and lives in the request's slot.
* feed-forward: sigmoid router, choice by score + correction, weights = scores * scale (not renormalised), experts
  down(relu(up h)^2).

The forward runs one ragged batch (``layer_ops.RaggedBatch``): portions of prompts and single decoded tokens side by side, over
``engine.state_cache.PagedStateCache``.  Dense products are torch's (hipBLASLt / rocBLAS); everything else is a launch of
``libjf_layers.so``.  With float32 weights every product is a true 32-bit one."""
from __future__ import annotations

import json
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Dict, List, Optional

import numpy as np
import torch
import torch.nn.functional as F

from .. import layer_ops as LO
from ..engine.state_cache import PagedStateCache, RunSpec


@dataclass
class LokizenConfig:
    vocab_size: int
    hidden_size: int
    layers: List[Dict[str, Any]]
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    norm_eps: float = 1e-5
    embedding_scale: float = 1.0
    max_position_embeddings: int = 1 << 20          # the design has no limit of its own: the engine's max_model_len decides
    eos_token_id: int = -1
    pad_token_id: int = 0
    family: str = "ragged"

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LokizenConfig":
        lp = d.get("loop") or {}
        n = len(d["layers"])
        start, stop, times = int(lp.get("start", 0)), int(lp.get("stop", 0)), int(lp.get("times", 1))
        if not (0 <= start <= stop <= n) or times < 1:
            raise ValueError(f"loop {lp} does not fit {n} layers")
        for i, L in enumerate(d["layers"]):
            if L["type"] not in ("attention", "retention"):
                raise ValueError(f"layer {i}: unknown mixer {L['type']!r}")
            if L.get("mlp") is not None and L["mlp"].get("kind", "moe") != "moe":
                raise ValueError(f"layer {i}: unknown feed-forward {L['mlp'].get('kind')!r}")
        return cls(vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), layers=d["layers"], loop_start=start, loop_stop=stop,
                   loop_times=times, norm_eps=float(d["norm"]["eps"]), embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
                   eos_token_id=int(d.get("eos_token_id", -1)), pad_token_id=int(d.get("pad_token_id", 0)))

    @classmethod
    def from_json(cls, path) -> "LokizenConfig":
        return cls.from_dict(json.loads(Path(path).read_text()))

    def runs(self) -> List[tuple]:
        """(layer index, add the embedding output first?) in execution order."""
        a, b = self.loop_start, self.loop_stop
        out = [(i, False) for i in range(a)]
        for p in range(self.loop_times if b > a else 0):
            out += [(i, p > 0 and i == a) for i in range(a, b)]
        return out + [(i, False) for i in range(b, len(self.layers))]


def distance_bucket_table(rows: int, far: float, length: int) -> np.ndarray:
    """Row of a distance-bias table for every distance 0 .. length-1: distances below rows/2 have a row each, then
    half + floor(ln(n / half) / ln(far / half) * (rows - half)), capped at the last row.  Evaluated once on the host in
    float32, so that every launch and every portion of a prompt agrees on the edges."""
    half = rows // 2
    n = np.arange(length, dtype=np.int64)
    out = n.copy()
    big = n >= half
    if big.any():
        f = np.float32
        with np.errstate(divide="ignore", invalid="ignore"):
            step = np.log(n[big].astype(f) / f(half)) / np.log(f(far) / f(half)) * f(rows - half)
        # a table whose far distance is not beyond its half has no logarithmic part: everything from the half on is the last row
        step = np.nan_to_num(np.floor(step), nan=float(rows), posinf=float(rows), neginf=0.0)
        out[big] = np.clip(half + step.astype(np.int64), half, rows - 1)
    return out.astype(np.int32)


class LokizenWeights:
    """Tensors by their checkpoint names (``embed``, ``l<i>.norm1``, ``l<i>.mix.q`` …, ``final.norm``, ``head``), regrouped per
    layer for the forward: the mixer's input projections stacked into one matrix, the experts stacked into [E, ff, W] / [E, W, ff],
    the small tables (distance bias, head mixing, router, correction, decay) in float."""

    def __init__(self, cfg: LokizenConfig, tensors: Dict[str, torch.Tensor], device, dtype=torch.bfloat16):
        dev = torch.device(device)
        act = lambda k: tensors[k].to(device=dev, dtype=dtype).contiguous()
        f32 = lambda k: tensors[k].to(device=dev, dtype=torch.float32).contiguous()
        self.device, self.dtype = dev, dtype
        self.embed, self.final_norm, self.head = act("embed"), act("final.norm"), act("head")
        if tuple(self.embed.shape) != (cfg.vocab_size, cfg.hidden_size):
            raise ValueError(f"embed is {tuple(self.embed.shape)}, config says {(cfg.vocab_size, cfg.hidden_size)}")
        self.layers = []
        for i, L in enumerate(cfg.layers):
            p, m = f"l{i}.", L["mixer"]
            w = dict(type=L["type"], norm1=act(p + "norm1"), w_o=act(p + "mix.o"))
            if L["type"] == "attention":
                H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
                if H % G:
                    raise ValueError(f"layer {i}: {H} heads over {G} key/value heads")
                w.update(w_in=torch.cat([act(p + "mix.q"), act(p + "mix.k"), act(p + "mix.v"), act(p + "mix.g")], 0),
                         cols=(0, H * D, H * D + G * D, H * D + G * D + G * Dv), q_norm=act(p + "mix.q.norm"), k_norm=act(p + "mix.k.norm"),
                         rel=f32(p + "mix.rel"), talk=f32(p + "mix.talk"))
                if tuple(w["talk"].shape) != (H, H) or w["rel"].shape[1] != H:
                    raise ValueError(f"layer {i}: head-mixing / distance-bias tables do not fit {H} heads")
                want = H * D + G * D + G * Dv + H * Dv
            else:
                H, D, Dv = m["heads"], m["dim"], m["vdim"]
                w.update(w_in=torch.cat([act(p + "mix.q"), act(p + "mix.k"), act(p + "mix.v"), act(p + "mix.g")], 0),
                         cols=(0, H * D, 2 * H * D, 2 * H * D + H * Dv), decay=torch.tensor(m["decay"], dtype=torch.float32, device=dev))
                if len(m["decay"]) != H:
                    raise ValueError(f"layer {i}: {len(m['decay'])} decays for {H} heads")
                want = 2 * H * D + 2 * H * Dv
            if w["w_in"].shape[0] != want:
                raise ValueError(f"layer {i}: projections have {w['w_in'].shape[0]} rows, the config's sizes give {want}")
            if L.get("mlp") is not None:
                E = L["mlp"]["router"]["experts"]
                w.update(norm2=act(p + "norm2"), router=f32(p + "mlp.router"), correction=f32(p + "mlp.correction"),
                         w_up=torch.stack([act(p + f"mlp.e{e}.up") for e in range(E)]).contiguous(),
                         w_down=torch.stack([act(p + f"mlp.e{e}.down") for e in range(E)]).contiguous())
            self.layers.append(w)

    @classmethod
    def from_safetensors(cls, cfg: LokizenConfig, model_dir, device, dtype=torch.bfloat16) -> "LokizenWeights":
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
    def random(cls, cfg: LokizenConfig, device, dtype=torch.bfloat16, seed: int = 0) -> "LokizenWeights":
        return cls(cfg, random_tensors(cfg, seed), device, dtype)


def random_tensors(cfg: LokizenConfig, seed: int = 0, rel_rows: int = 16) -> Dict[str, torch.Tensor]:
    """Random tensors under the checkpoint's names (benchmarks and tests; bf16-representable float32 values)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg.hidden_size
    rnd = lambda *s, std=1.0: (torch.randn(*s, generator=g) * std).to(torch.bfloat16).float()
    lin = lambda o, i: rnd(o, i, std=i ** -0.5)
    one = lambda n: (1 + torch.randn(n, generator=g) * 0.1).to(torch.bfloat16).float()
    t = {"embed": rnd(cfg.vocab_size, W), "final.norm": one(W), "head": lin(cfg.vocab_size, W)}
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.", L["mixer"]
        t[p + "norm1"] = one(W)
        if L["type"] == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            t.update({p + "mix.q": lin(H * D, W), p + "mix.k": lin(G * D, W), p + "mix.v": lin(G * Dv, W), p + "mix.g": lin(H * Dv, W),
                      p + "mix.o": lin(W, H * Dv), p + "mix.q.norm": one(H * D), p + "mix.k.norm": one(G * D),
                      p + "mix.rel": rnd(rel_rows, H), p + "mix.talk": (torch.eye(H) + rnd(H, H, std=0.3)).to(torch.bfloat16).float()})
        else:
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            t.update({p + "mix.q": lin(H * D, W), p + "mix.k": lin(H * D, W), p + "mix.v": lin(H * Dv, W), p + "mix.g": lin(H * Dv, W),
                      p + "mix.o": lin(W, H * Dv)})
        if L.get("mlp") is not None:
            E, ff = L["mlp"]["router"]["experts"], L["mlp"]["expert"]["ff"]
            t[p + "norm2"] = one(W)
            t[p + "mlp.router"] = lin(E, W) * 2
            t[p + "mlp.correction"] = rnd(E, std=0.1)
            for e in range(E):
                t[p + f"mlp.e{e}.up"] = lin(ff, W)
                t[p + f"mlp.e{e}.down"] = lin(W, ff)
    return t


DIRECT_BIAS_POSITIONS = 1 << 16


class LokizenModel:
    def __init__(self, cfg: LokizenConfig, weights: LokizenWeights, max_positions: int = 8192):
        self.cfg, self.w = cfg, weights
        self.device, self.dtype = weights.device, weights.dtype
        self.runs = cfg.runs()
        self.readd = any(r for _, r in self.runs)
        self._angles: Dict[tuple, tuple] = {}
        self._luts: Dict[tuple, torch.Tensor] = {}
        self.max_positions = 0
        self.reserve_positions(max_positions)

    # ---- what the cache must hold, one entry per layer run -----------------------------------------------------------------------
    def cache_specs(self) -> List[RunSpec]:
        specs = []
        for li, _ in self.runs:
            L, m = self.cfg.layers[li], self.cfg.layers[li]["mixer"]
            if L["type"] == "attention":
                specs.append(RunSpec("kv", k_width=m["kv_heads"] * m["dim"], v_width=m["kv_heads"] * m["vdim"]))
            else:
                specs.append(RunSpec("state", state_shape=(m["heads"], m["dim"], m["vdim"])))
        return specs

    def new_cache(self, num_pages: int, page_size: int, num_slots: int) -> PagedStateCache:
        return PagedStateCache(self.cache_specs(), num_pages, page_size, num_slots, self.device, self.dtype)

    # ---- position tables: rotation angles and distance buckets, for every position the engine can reach --------------------------
    def reserve_positions(self, n: int) -> None:
        if n <= self.max_positions:
            return
        self.max_positions = int(n)
        self._angles.clear()
        self._luts.clear()
        self._bias = {}
        for i, L in enumerate(self.cfg.layers):
            m = L["mixer"]
            if L["type"] == "retention":
                rot = m.get("rot") or {}
                dims, base = int(rot.get("dims", 0)), float(rot.get("base", 10000.0))
                if dims and (dims, base) not in self._angles:
                    f = torch.tensor([base ** (-2.0 * k / dims) for k in range(dims // 2)], dtype=torch.float32, device=self.device)
                    a = torch.arange(n, dtype=torch.float32, device=self.device).view(n, 1) * f.view(1, -1)
                    self._angles[(dims, base)] = (a.cos().contiguous(), a.sin().contiguous())
            else:
                key = (int(self.w.layers[i]["rel"].shape[0]), float(m["bias_max"]))
                if key not in self._luts:
                    self._luts[key] = torch.from_numpy(distance_bucket_table(key[0], key[1], n)).to(self.device)
                # up to DIRECT_BIAS_POSITIONS the bias is laid out by distance, [positions, H]: one lookup per score instead of two
                self._bias[i] = self.w.layers[i]["rel"][self._luts[key].long()].contiguous() if n <= DIRECT_BIAS_POSITIONS else None

    # ---- mixers ---------------------------------------------------------------------------------------------------------------
    def _attention(self, run: int, li: int, h: torch.Tensor, batch: LO.RaggedBatch, cache: PagedStateCache) -> torch.Tensor:
        m, w, eps = self.cfg.layers[li]["mixer"], self.w.layers[li], self.cfg.norm_eps
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        proj = F.linear(h, w["w_in"])
        q = LO.qk_norm_append(proj, w["cols"][:3], H, G, D, Dv, w["q_norm"], w["k_norm"], eps, cache.k[run], cache.v[run], batch.kv_slot)
        gate = proj[:, w["cols"][3]:w["cols"][3] + H * Dv]
        mask = m.get("mask") or {}
        direct = self._bias.get(li)
        rel, lut = (direct, None) if direct is not None else (w["rel"], self._luts[(int(w["rel"].shape[0]), float(m["bias_max"]))])
        return LO.attn_window(q, gate, cache.k[run], cache.v[run], batch, H, G, D, Dv, m["scale"], int(mask.get("size", 0)),
                              int(mask.get("keep_first", 0)), rel, lut, w["talk"])

    def _retention(self, run: int, li: int, h: torch.Tensor, batch: LO.RaggedBatch, cache: PagedStateCache) -> torch.Tensor:
        m, w = self.cfg.layers[li]["mixer"], self.w.layers[li]
        rot = m.get("rot") or {}
        dims = int(rot.get("dims", 0))
        cos, sin = self._angles[(dims, float(rot.get("base", 10000.0)))] if dims else (None, None)
        return LO.retention(F.linear(h, w["w_in"]), w["cols"], batch, m["heads"], m["dim"], m["vdim"], dims, cos, sin, w["decay"],
                            self.cfg.norm_eps, cache.state[run])

    # ---- one step ----------------------------------------------------------------------------------------------------------------
    @torch.inference_mode()
    def forward(self, ids: torch.Tensor, batch: LO.RaggedBatch, cache: PagedStateCache, logit_rows: Optional[torch.Tensor] = None,
                trace: Optional[list] = None) -> torch.Tensor:
        """ids int64 [N] (the batch's rows).  Returns float logits [N, vocab], or of the rows in ``logit_rows``.  ``trace``, when a
        list, receives the residual stream after every layer run (debugging and tests)."""
        cfg, w, eps, dt = self.cfg, self.w, self.cfg.norm_eps, self.dtype
        if batch.max_pos > self.max_positions:
            raise ValueError(f"position {batch.max_pos - 1} is beyond the {self.max_positions} positions the tables were reserved for")
        x, x0 = LO.embed_scale(w.embed, ids, cfg.embedding_scale, self.readd)
        pending = None                                   # a mixer's or feed-forward's output, folded into the next norm's launch
        for run, (li, readd) in enumerate(self.runs):
            L, lw = cfg.layers[li], w.layers[li]
            h = LO.add_rmsnorm(x, pending, x0 if readd else None, lw["norm1"], eps, dt)
            a = self._attention(run, li, h, batch, cache) if L["type"] == "attention" else self._retention(run, li, h, batch, cache)
            pending = F.linear(a, lw["w_o"])
            if L.get("mlp") is not None:
                r = L["mlp"]["router"]
                h2 = LO.add_rmsnorm(x, pending, None, lw["norm2"], eps, dt)
                pending = LO.moe_experts(h2, F.linear(h2.float(), lw["router"]), lw["correction"], int(r["top"]), float(r["scale"]),
                                         lw["w_up"], lw["w_down"])
            if trace is not None:
                LO.add_rmsnorm(x, pending, None, None, eps, None)
                pending = None
                trace.append(x.clone())
        hf = LO.add_rmsnorm(x, pending, None, w.final_norm, eps, dt)
        if logit_rows is not None:
            hf = hf.index_select(0, logit_rows)
        return F.linear(hf, w.head).float()


def load_model_directory(model_dir, device, dtype=torch.bfloat16, max_positions: int = 8192):
    cfg = LokizenConfig.from_json(Path(model_dir) / "config.json")
    return cfg, LokizenModel(cfg, LokizenWeights.from_safetensors(cfg, model_dir, device, dtype), max_positions)


def random_model(cfg: LokizenConfig, device, dtype=torch.bfloat16, max_positions: int = 8192, seed: int = 0) -> LokizenModel:
    return LokizenModel(cfg, LokizenWeights.random(cfg, device, dtype, seed), max_positions)
