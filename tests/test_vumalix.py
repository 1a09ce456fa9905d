"""Vumalix through the package (HIP layer kernels, paged pools + convolution tails in state slots, ragged step, scheduler,
LLM.generate) against the plain oracle ``oracle/vumalix_oracle.py``, which shares no code with it.  Small random models of several
shapes; where random weights would hide a fault (a key at a window's edge, a far key among hundreds) the inputs are chosen so
that one score stands out.

CPU tests cover the oracle's own pieces, the config reader and the cache layout; everything that launches a kernel is marked
``gpu``."""
import json
import math
import random

import numpy as np
import pytest
import torch

from oracle import vumalix_oracle as O
from jacobiforcing_amd.modeling import MODEL_REGISTRY, read_model_config
from jacobiforcing_amd.modeling import vumalix as VX

gpu = pytest.mark.gpu


# ---- model shapes -----------------------------------------------------------------------------------------------------------------
def diff_attn(heads=6, kv=2, dim=24, vdim=40, diff=0.3, coef=0.4, every=5, scale=0.3):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff,
                                           "q_temp": {"coef": coef, "every": every}}}


def latent(heads=3, dim=24, rot_dim=16, vdim=40, kv_rank=48, q_rank=36, size=11, base=500.0, scale=0.2, dims=None):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
                                                  "scale": scale, "mask": {"size": size}, "rot": {"dims": rot_dim if dims is None else dims, "base": base}}}


def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def make_cfg(layers, width=96, vocab=131, taps=3, eps=1e-5):
    return {"architecture": "Vumalix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "canon": {"taps": taps}, "layers": layers}


def shape_a():
    """Both mixers, a layer without feed-forward, borrowed weights of either mixer, grouped key/value heads, three taps."""
    return make_cfg([dict(latent(), mlp=dense()), dict(diff_attn(), mlp=dense(40)), dict(latent(), mlp=dense(), weights_of=0),
                     dict(diff_attn(heads=4, kv=4, dim=16, vdim=16, diff=0.8, coef=0.0), mlp=None), dict(diff_attn(), mlp=dense(40), weights_of=1)])


def shape_b():
    """One head, one key/value head for several query heads, a window of one page, five taps, a temperature step at every token,
    sizes that are no multiples of eight."""
    return make_cfg([dict(diff_attn(heads=1, kv=1, dim=20, vdim=72, diff=0.5, coef=1.0, every=1), mlp=dense(24)),
                     dict(latent(heads=1, dim=12, rot_dim=8, vdim=20, kv_rank=28, q_rank=20, size=8, base=10000.0), mlp=dense(33)),
                     dict(diff_attn(heads=3, kv=1, dim=32, vdim=24, diff=0.1, coef=0.2, every=64), mlp=None)],
                    width=64, vocab=77, taps=5, eps=1e-6)


def shape_c():
    """No convolution beyond the token itself (one tap), a window longer than any test sequence, many heads."""
    return make_cfg([dict(latent(heads=10, dim=16, rot_dim=8, vdim=16, kv_rank=32, q_rank=24, size=4096), mlp=dense(48)),
                     dict(diff_attn(heads=10, kv=5, dim=16, vdim=16), mlp=dense(48))], width=80, vocab=50, taps=1)


SHAPES = {"a": shape_a, "b": shape_b, "c": shape_c}


def tensors_for(cfg_dict, seed):
    return VX.random_tensors(VX.VumalixConfig.from_dict(cfg_dict), seed)


def rel_err(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    return float(np.sqrt(((got - want) ** 2).mean()) / max(np.sqrt((want ** 2).mean()), 1e-30))


F32_TOL, BF16_TOL = 2e-4, 6e-2


def toks(n, vocab, seed):
    return [random.Random(seed * 7919 + i).randrange(vocab) for i in range(n)]


# =====================================================================================================================================
# CPU: oracle pieces, config reader, cache layout
# =====================================================================================================================================
def test_registry_reads_the_architecture_key(tmp_path):
    assert MODEL_REGISTRY["Vumalix"][2] == "ragged"
    (tmp_path / "config.json").write_text(json.dumps(shape_a()))
    cfg = read_model_config(tmp_path)
    assert isinstance(cfg, VX.VumalixConfig) and cfg.family == "ragged" and cfg.conv_taps == 3 and cfg.num_hidden_layers == 5
    assert [cfg.weights_layer(i) for i in range(5)] == [0, 1, 0, 3, 1]


def test_config_rejects_what_the_design_does_not_have():
    bad = shape_a()
    bad["layers"][2]["weights_of"] = 1                                                        # a latent layer borrowing attention weights
    with pytest.raises(ValueError):
        VX.VumalixConfig.from_dict(bad)
    bad = shape_a()
    bad["layers"][0]["type"] = "retention"
    with pytest.raises(ValueError):
        VX.VumalixConfig.from_dict(bad)
    bad = shape_a()
    bad["layers"][1]["mlp"]["kind"] = "moe"
    with pytest.raises(ValueError):
        VX.VumalixConfig.from_dict(bad)
    chain = shape_a()
    chain["layers"][4]["weights_of"] = 2                                                       # borrows from a layer that borrows: followed
    assert VX.VumalixConfig.from_dict(dict(chain, layers=chain["layers"][:3] + [chain["layers"][0] | {"weights_of": 2}])).weights_layer(3) == 0
    bad = shape_a()
    bad["canon"]["taps"] = 0
    with pytest.raises(ValueError):
        VX.VumalixConfig.from_dict(bad)


def test_borrowed_weights_are_shared_and_caches_are_not():
    cfg = VX.VumalixConfig.from_dict(shape_a())
    w = VX.VumalixWeights(cfg, tensors_for(shape_a(), 1), "cpu", torch.float32)
    assert w.layers[2] is w.layers[0] and w.layers[4] is w.layers[1] and w.layers[3] is not w.layers[1]
    assert "l2.mix.dq" not in tensors_for(shape_a(), 1)
    specs = VX.VumalixModel(cfg, w, max_positions=16).cache_specs()
    assert len(specs) == 5 and all(s.kind == "kv" and s.tail_shape == (2, 96) for s in specs)
    assert (specs[0].k_width, specs[0].v_width) == (48 + 16, 0) and (specs[1].k_width, specs[1].v_width) == (2 * 2 * 24, 2 * 40)
    from jacobiforcing_amd.engine.state_cache import PagedStateCache
    cache = PagedStateCache(specs, 4, 8, 3, "cpu", torch.float32)
    assert cache.v[0] is None and tuple(cache.k[0].shape) == (32, 64) and tuple(cache.tail[4].shape) == (3, 2, 96)
    one_tap = VX.VumalixModel(VX.VumalixConfig.from_dict(shape_c()), VX.VumalixWeights(VX.VumalixConfig.from_dict(shape_c()), tensors_for(shape_c(), 1),
                                                                                         "cpu", torch.float32), 16)
    assert PagedStateCache(one_tap.cache_specs(), 4, 8, 3, "cpu", torch.float32).tail[0] is None


def test_oracle_convolution_and_rotation():
    x = torch.arange(12, dtype=torch.float64).view(6, 2) + 1
    w = torch.tensor([[0.5, 0.25, 2.0], [0.0, 0.0, 1.0]], dtype=torch.float64)
    y = O.time_conv_mix(x, w)
    assert torch.allclose(y[:, 1], 2 * x[:, 1])                                               # the last tap is the token itself
    assert float(y[0, 0]) == 1 + 2 * 1 and float(y[2, 0]) == 5 + 0.5 * 1 + 0.25 * 3 + 2 * 5     # zeros before the start
    v = torch.tensor([1.0, 2.0, 3.0, 4.0, 5.0, 6.0], dtype=torch.float64)
    r = O.rotate_pairs(v, 3, 4, 100.0)
    a0, a1 = 3.0, 3.0 * 100.0 ** -0.5
    assert abs(float(r[0]) - (1 * math.cos(a0) - 3 * math.sin(a0))) < 1e-6 and abs(float(r[3]) - (4 * math.cos(a1) + 2 * math.sin(a1))) < 1e-6
    assert float(r[4]) == 5.0 and float(r[5]) == 6.0 and torch.equal(O.rotate_pairs(v, 0, 4, 100.0), v)
    # turning query and key by their positions leaves a score that depends on the distance only
    q, k = torch.randn(8, dtype=torch.float64), torch.randn(8, dtype=torch.float64)
    s1 = O.rotate_pairs(q, 9, 8, 50.0) @ O.rotate_pairs(k, 4, 8, 50.0)
    s2 = O.rotate_pairs(q, 25, 8, 50.0) @ O.rotate_pairs(k, 20, 8, 50.0)
    assert abs(float(s1 - s2)) < 1e-5


def test_oracle_temperature_lambda_and_activation():
    assert O.query_temperature(0, 0.5, 4) == 1.0 and O.query_temperature(2, 0.5, 4) == 1.0
    assert abs(O.query_temperature(3, 0.5, 4) - (1 + 0.5 * math.log(2))) < 1e-12 and abs(O.query_temperature(11, 2.0, 4) - (1 + 2 * math.log(4))) < 1e-12
    P = {"mix.lq1": torch.tensor([1.0, 2.0]), "mix.lk1": torch.tensor([0.5, 0.25]), "mix.lq2": torch.tensor([0.0, 1.0]), "mix.lk2": torch.tensor([3.0, -1.0])}
    assert abs(O.differential_lambda(P, 0.3) - (math.e - math.exp(-1) + 0.3)) < 1e-6
    z = torch.tensor([[1.0, -2.0, 3.0, 0.5]], dtype=torch.float64)
    got = O.polynomial_activation(z, torch.tensor([2.0, 0.0, 0.0, 0.25], dtype=torch.float64), 0.0)
    assert torch.allclose(got, 2 * z / math.sqrt(float((z * z).mean())) + 0.25)
    got = O.polynomial_activation(z, torch.tensor([0.0, 0.0, 1.0, 0.0], dtype=torch.float64), 0.0)
    assert abs(float((got * got).mean()) - 1.0) < 1e-12 and torch.allclose(got / got[0, 0], z ** 3)


def test_oracle_latent_attention_equals_the_query_side_form():
    """Scores and outputs through keys / values built per token equal those with the up-projections moved to the query and to the
    output: the identity the package's kernels rely on."""
    cfg = make_cfg([dict(latent(size=5), mlp=None)])
    m, P = cfg["layers"][0]["mixer"], {k: v.double() for k, v in O.layer_tensors(tensors_for(cfg, 2), 0).items()}
    T, eps = 9, cfg["norm"]["eps"]
    h = torch.randn(T, 96, dtype=torch.float64, generator=torch.Generator().manual_seed(0))
    want = O.latent_attention(h, P, m, eps)
    H, D, rd, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = ((O.unit_rms(h @ P["mix.dq"].T, eps) * P["mix.dq.norm"]) @ P["mix.uq"].T).view(T, H, D + rd)
    down = h @ P["mix.dkv"].T
    lat = O.unit_rms(down[:, :R], eps) * P["mix.dkv.norm"]
    uk, uv = P["mix.uk"].view(H, D, R), P["mix.uv"].view(H, Dv, R)
    out = torch.zeros(T, H, Dv, dtype=torch.float64)
    for i in range(T):
        lo = max(0, i - 4)
        for hh in range(H):
            qa = q[i, hh, :D] @ uk[hh]
            s = torch.stack([(qa @ lat[j] + O.rotate_pairs(q[i, hh, D:], i, rd, 500.0) @ O.rotate_pairs(down[j, R:], j, rd, 500.0)) * m["scale"]
                             for j in range(lo, i + 1)])
            out[i, hh] = uv[hh] @ (torch.softmax(s, 0) @ lat[lo:i + 1])
    got = (out.reshape(T, H * Dv) * torch.sigmoid(h @ P["mix.g"].T)) @ P["mix.o"].T
    assert rel_err(got, want) < 1e-12


# =====================================================================================================================================
# GPU: the package against the oracle
# =====================================================================================================================================
class Rig:
    """A model on the GPU with a pool of shuffled pages; runs steps of (request, tokens) and keeps the bookkeeping a test needs."""

    def __init__(self, cfg_dict, seed=0, dtype=torch.float32, page=8, pages=64, slots=4, tensors=None):
        from jacobiforcing_amd import layer_ops as LO
        self.LO = LO
        self.cfg_dict = cfg_dict
        self.cfg = VX.VumalixConfig.from_dict(cfg_dict)
        self.tensors = tensors or tensors_for(cfg_dict, seed)
        self.model = VX.VumalixModel(self.cfg, VX.VumalixWeights(self.cfg, self.tensors, "cuda", dtype), max_positions=1024)
        self.page = page
        self.cache = self.model.new_cache(pages, page, slots)
        self.free_pages = list(range(pages))
        random.Random(seed).shuffle(self.free_pages)
        self.free_slots = list(range(slots))[::-1]
        self.req = {}

    def poison(self):
        """Fill pools and tails with large values: whatever a kernel reads without having written it shows."""
        for t in self.cache.k + self.cache.v + self.cache.tail:
            if t is not None:
                t.fill_(1e4)

    def step(self, entries, trace=None):
        """entries = [(key, tokens)]; returns logits [sum of tokens, vocab] (float, on the CPU)."""
        counts, starts, slots, tables, ids = [], [], [], [], []
        for key, tk in entries:
            r = self.req.setdefault(key, {"n": 0, "pages": [], "slot": None})
            if r["slot"] is None:
                r["slot"] = self.free_slots.pop()
            while len(r["pages"]) * self.page < r["n"] + len(tk):
                r["pages"].append(self.free_pages.pop())
            counts.append(len(tk)); starts.append(r["n"]); slots.append(r["slot"]); tables.append(r["pages"])
            ids += list(tk)
            r["n"] += len(tk)
        b = self.LO.RaggedBatch.build(counts, starts, slots, tables, self.page, "cuda")
        return self.model.forward(torch.tensor(ids, device="cuda"), b, self.cache, None, trace).cpu()

    def end(self, key):
        r = self.req.pop(key)
        self.free_pages += r["pages"][::-1]
        self.free_slots.append(r["slot"])

    def oracle(self, tokens):
        return O.forward(self.cfg_dict, self.tensors, list(tokens), torch.float64)


@gpu
@pytest.mark.parametrize("W", [96, 200, 1000])
def test_output_norm_residual_and_activation(W):
    from jacobiforcing_amd import layer_ops as LO
    g = torch.Generator().manual_seed(W)
    x, y, gw = torch.randn(5, W, generator=g), torch.randn(5, W, generator=g) * 3, torch.tensor([0.7])
    want = x.double() + O.unit_rms(y.double(), 1e-5) * 0.7
    xd = x.cuda()
    out = LO.norm_add(xd, y.cuda(), gw.cuda(), 1e-5, torch.float32)
    assert rel_err(xd.cpu(), want) < 1e-6 and rel_err(out.cpu(), want) < 1e-6
    xb = x.cuda()
    outb = LO.norm_add(xb, y.cuda().bfloat16(), gw.cuda(), 1e-5, torch.bfloat16)
    wantb = x.double() + O.unit_rms(y.bfloat16().double(), 1e-5) * 0.7
    assert xb.dtype == torch.float32 and rel_err(xb.cpu(), wantb) < 1e-6 and rel_err(outb.float().cpu(), wantb) < 6e-3
    assert LO.norm_add(xb, y.cuda(), gw.cuda(), 1e-5, None) is None
    tiny = torch.full((1, W), 1e-4)                                                            # eps inside the root decides here
    xt = torch.zeros(1, W).cuda()
    LO.norm_add(xt, tiny.cuda(), gw.cuda(), 1e-5, None)
    assert rel_err(xt.cpu(), O.unit_rms(tiny.double(), 1e-5) * 0.7) < 1e-6
    coef = torch.tensor([0.5, -1.25, 0.75, 0.1])
    z = torch.randn(7, W, generator=g) * 2
    assert rel_err(LO.polynorm(z.cuda(), coef.cuda(), 1e-6).cpu(), O.polynomial_activation(z.double(), coef.double(), 1e-6)) < 1e-6
    zb = z.bfloat16()
    assert rel_err(LO.polynorm(zb.cuda(), coef.cuda(), 1e-6).float().cpu(), O.polynomial_activation(zb.double(), coef.double(), 1e-6)) < 6e-3


@gpu
@pytest.mark.parametrize("taps,cuts", [(4, [9]), (4, [1, 1, 1, 2, 4]), (3, [2, 7]), (7, [3, 2, 1, 3]), (1, [4, 5]), (2, [1] * 9), (9, [3, 5, 1, 1, 12]),
                                       (5, [1, 19, 2, 1, 1])])
def test_convolution_carries_its_tail_across_steps(taps, cuts):
    """A request cut into portions shorter and longer than the taps, beside a second request that starts later in a used slot.
    Width 70 takes the kernel with a channel per thread, 72 the one with four channels per thread and the inputs kept in registers
    (up to eight taps)."""
    from jacobiforcing_amd import layer_ops as LO
    for W in (70, 72):
        T = sum(cuts)
        g = torch.Generator().manual_seed(taps)
        xa, xb, w = torch.randn(T, W, generator=g), torch.randn(T, W, generator=g), torch.randn(W, taps, generator=g)
        want_a, want_b = O.time_conv_mix(xa.double(), w.double()), O.time_conv_mix(xb[:T - cuts[0]].double(), w.double())
        tail = torch.full((3, taps - 1, W), 1e4).cuda() if taps > 1 else None
        got_a, got_b, done = [], [], 0
        for s, c in enumerate(cuts):
            counts, starts, slots, rows = [c], [done], [2], [xa[done:done + c]]
            if s > 0:                                                                          # the second request is one portion behind
                counts.append(c); starts.append(done - cuts[0]); slots.append(0); rows.append(xb[done - cuts[0]:done - cuts[0] + c])
            b = LO.RaggedBatch.build(counts, starts, slots, [[0, 1, 2, 3]] * len(counts), 16, "cuda")
            out = LO.causal_conv(torch.cat(rows).cuda(), w.cuda(), b, tail).cpu()
            got_a.append(out[:c])
            if s > 0:
                got_b.append(out[c:])
            done += c
        assert rel_err(torch.cat(got_a), want_a) < 1e-6, W
        if got_b:
            assert rel_err(torch.cat(got_b), want_b[:sum(cuts[1:])]) < 1e-6, W


@gpu
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_each_mixer_and_feed_forward_alone(name):
    """Layer by layer on the oracle's own inputs: mixer output (through the output projection) and feed-forward for a whole prompt."""
    import torch.nn.functional as F
    rig = Rig(SHAPES[name](), seed=3)
    T = 37
    h = torch.randn(T, rig.cfg.hidden_size, generator=torch.Generator().manual_seed(1))
    b = rig.LO.RaggedBatch.build([T], [0], [1], [[9, 3, 20, 11, 5]], 8, "cuda")
    for li, L in enumerate(rig.cfg_dict["layers"]):
        P = {k: v.double() for k, v in O.layer_tensors(rig.tensors, L.get("weights_of", li)).items()}
        lw = rig.model.w.layers[li]
        if L["type"] == "attention":
            got, want = rig.model._attention(li, h.cuda(), b, rig.cache), O.differential_attention(h.double(), P, L["mixer"], rig.cfg.norm_eps)
        else:
            got, want = rig.model._latent_attention(li, h.cuda(), b, rig.cache), O.latent_attention(h.double(), P, L["mixer"], rig.cfg.norm_eps)
        assert rel_err(F.linear(got, lw["w_o"]).cpu(), want) < 1e-5, (li, L["type"])
        if L.get("mlp"):
            y = F.linear(rig.LO.polynorm(F.linear(h.cuda(), lw["w_up"]), lw["act"], rig.cfg.norm_eps), lw["w_down"])
            assert rel_err(y.cpu(), O.feed_forward(h.double(), P, rig.cfg.norm_eps)) < 1e-5, li


@gpu
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_whole_prompt_and_every_layer(name):
    rig = Rig(SHAPES[name](), seed=5)
    t = toks(61, rig.cfg.vocab_size, 1)
    trace = []
    got = rig.step([("p", t)], trace)
    want, want_trace = rig.oracle(t)
    assert len(trace) == want_trace.shape[0]
    for i, x in enumerate(trace):
        assert rel_err(x.cpu(), want_trace[i]) < 1e-5, f"layer {i}"
    assert rel_err(got, want) < F32_TOL
    assert rel_err(Rig(SHAPES[name](), seed=5, dtype=torch.bfloat16).step([("p", t)]), want) < BF16_TOL


@gpu
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_prefill_equals_token_by_token_decoding(name):
    rig = Rig(SHAPES[name](), seed=7)
    t = toks(40, rig.cfg.vocab_size, 2)
    want, _ = rig.oracle(t)
    rig.poison()
    whole = rig.step([("whole", t)])
    single = torch.cat([rig.step([("single", [x])]) for x in t])
    assert rel_err(whole, want) < F32_TOL and rel_err(single, want) < F32_TOL and rel_err(single, whole) < F32_TOL


@gpu
@pytest.mark.parametrize("cuts", [[2] * 20, [1, 2, 3, 5, 8, 13, 7, 1], [7, 9, 8, 16], [39, 1], [3, 37]])
def test_portions_of_any_size(cuts):
    """Cuts inside pages, windows and the convolution's reach; portions of two tokens."""
    for name in ("a", "b"):
        rig = Rig(SHAPES[name](), seed=11)
        t = toks(sum(cuts), rig.cfg.vocab_size, 3)
        want, _ = rig.oracle(t)
        rig.poison()
        got, at = [], 0
        for c in cuts:
            got.append(rig.step([("r", t[at:at + c])]))
            at += c
        assert rel_err(torch.cat(got), want) < F32_TOL, name


@gpu
@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 32, 48), (8, 8, 64, 32), (3, 1, 24, 40), (2, 1, 128, 128), (12, 4, 16, 16), (16, 4, 64, 128), (5, 5, 40, 96),
                                      (40, 1, 16, 32), (6, 2, 24, 160), (2, 1, 256, 512)])
def test_bfloat16_differential_attention_alone(H, G, D, Dv):
    """The bfloat16 paths — the one-sweep kernel where the value width is a multiple of 32 (groups of 1, 3, 4 and 40 heads), the
    two-sweep matrix-core kernel, one launch per map with many heads, the plain kernel for the rest — on a prompt of several tiles,
    then single tokens, against the oracle on the same bfloat16-rounded inputs."""
    import torch.nn.functional as F
    cfg = make_cfg([dict(diff_attn(heads=H, kv=G, dim=D, vdim=Dv, scale=D ** -0.5, every=16), mlp=None)], width=64)
    rig = Rig(cfg, seed=H, dtype=torch.bfloat16, page=16)
    T = 150
    h = (torch.randn(T, 64, generator=torch.Generator().manual_seed(2))).bfloat16()
    P = {k: v.double() for k, v in O.layer_tensors(rig.tensors, 0).items()}
    want = O.differential_attention(h.double(), P, cfg["layers"][0]["mixer"], 1e-5)
    pages = list(range(20, 30))
    b = rig.LO.RaggedBatch.build([T - 3], [0], [0], [pages], 16, "cuda")
    got = [F.linear(rig.model._attention(0, h[:T - 3].cuda(), b, rig.cache), rig.model.w.layers[0]["w_o"])]
    for i in range(T - 3, T):
        b = rig.LO.RaggedBatch.build([1], [i], [0], [pages], 16, "cuda")
        got.append(F.linear(rig.model._attention(0, h[i:i + 1].cuda(), b, rig.cache), rig.model.w.layers[0]["w_o"]))
    assert rel_err(torch.cat(got).float().cpu(), want) < 3e-2


@gpu
@pytest.mark.parametrize("H,D,rd,Dv,R,size", [(6, 64, 32, 48, 96, 50), (4, 32, 16, 48, 64, 20), (16, 16, 8, 16, 32, 33), (2, 24, 8, 20, 200, 40),
                                               (20, 16, 16, 16, 48, 17), (6, 48, 16, 40, 128, 50), (16, 32, 32, 32, 256, 33), (40, 16, 8, 16, 128, 20),
                                               (3, 24, 8, 20, 384, 70), (1, 16, 64, 24, 512, 1000), (5, 16, 8, 16, 128, 1)])
def test_bfloat16_latent_attention_alone(H, D, rd, Dv, R, size):
    """Latents of 128, 256, 384 and 512 take the one-sweep kernel for a shared key/value head (1, 3, 5, 6, 16 and 40 heads: part of
    a row tile, a whole one, two of them); the others the general kernels, 200 in two column ranges."""
    import torch.nn.functional as F
    cfg = make_cfg([dict(latent(heads=H, dim=D, rot_dim=rd, vdim=Dv, kv_rank=R, q_rank=40, size=size, scale=(D + rd) ** -0.5), mlp=None)], width=64)
    rig = Rig(cfg, seed=H, dtype=torch.bfloat16, page=16)
    T = 150
    h = (torch.randn(T, 64, generator=torch.Generator().manual_seed(3))).bfloat16()
    P = {k: v.double() for k, v in O.layer_tensors(rig.tensors, 0).items()}
    want = O.latent_attention(h.double(), P, cfg["layers"][0]["mixer"], 1e-5)
    pages = list(range(40, 50))
    b = rig.LO.RaggedBatch.build([T - 3], [0], [0], [pages], 16, "cuda")
    got = [F.linear(rig.model._latent_attention(0, h[:T - 3].cuda(), b, rig.cache), rig.model.w.layers[0]["w_o"])]
    for i in range(T - 3, T):
        b = rig.LO.RaggedBatch.build([1], [i], [0], [pages], 16, "cuda")
        got.append(F.linear(rig.model._latent_attention(0, h[i:i + 1].cuda(), b, rig.cache), rig.model.w.layers[0]["w_o"]))
    assert rel_err(torch.cat(got).float().cpu(), want) < 3e-2


@gpu
def test_unequal_requests_in_one_batch_equal_each_alone():
    rig = Rig(shape_a(), seed=13, pages=96)
    V = rig.cfg.vocab_size
    reqs = {"long": toks(70, V, 4), "mid": toks(23, V, 5), "one": toks(1, V, 6), "two": toks(2, V, 7)}
    want = {k: rig.oracle(v)[0] for k, v in reqs.items()}
    rig.poison()
    # step 1: portions of three prompts side by side; step 2: the rest of one, single tokens of the others, a new request
    s1 = rig.step([("long", reqs["long"][:50]), ("mid", reqs["mid"][:22]), ("one", reqs["one"])])
    s2 = rig.step([("long", reqs["long"][50:51]), ("two", reqs["two"]), ("mid", reqs["mid"][22:])])
    s3 = rig.step([("long", reqs["long"][51:])])
    got = {"long": torch.cat([s1[:50], s2[:1], s3]), "mid": torch.cat([s1[50:72], s2[3:4]]), "one": s1[72:73], "two": s2[1:3]}
    for k in reqs:
        assert rel_err(got[k], want[k]) < F32_TOL, k


@gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32_TOL), (torch.bfloat16, BF16_TOL)])
def test_freed_pages_and_slots_are_used_again(dtype, tol):
    """Two slots, a pool that holds two requests: requests end, their pages and slots go to new ones, old content must not leak —
    neither old keys nor the convolution tail of the slot's previous request."""
    rig = Rig(shape_a(), seed=17, pages=12, slots=2, dtype=dtype)
    V = rig.cfg.vocab_size
    rig.poison()
    for rnd in range(4):
        a, b = toks(40 + rnd, V, 20 + rnd), toks(17 + 3 * rnd, V, 30 + rnd)
        ga = rig.step([("a", a[:25]), ("b", b[:1])])                                           # b starts with a single token in a used slot
        gb = rig.step([("a", a[25:]), ("b", b[1:])])
        got_a = torch.cat([ga[:25], gb[:len(a) - 25]])
        got_b = torch.cat([ga[25:], gb[len(a) - 25:]])
        assert rel_err(got_a, rig.oracle(a)[0]) < tol and rel_err(got_b, rig.oracle(b)[0]) < tol, rnd
        used = set(rig.req["a"]["pages"]) | set(rig.req["b"]["pages"])
        rig.end("b"); rig.end("a")
        assert len(rig.free_pages) == 12 and len(used) >= 8


def peaked_latent_model(size, R=24):
    """One latent-attention layer, no feed-forward, a sharp softmax, a convolution and a rotary part too weak to matter.  Returns
    (cfg, tensors, hot query token, hot key token, scores): the pair of tokens whose unrotated score is the largest."""
    cfg = make_cfg([dict(latent(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=R, q_rank=24, size=size, scale=3.0), mlp=None)], width=32, vocab=40)
    t = tensors_for(cfg, 23)
    t["l0.canon1"] = t["l0.canon1"] * 0.02
    t["l0.mix.dkv"][R:] *= 0.05
    eps = cfg["norm"]["eps"]
    h = t["embed"].double()
    q = ((O.unit_rms(h @ t["l0.mix.dq"].double().T, eps) * t["l0.mix.dq.norm"].double()) @ t["l0.mix.uq"].double().T).view(40, 2, 24)[:, 0, :16]
    lat = O.unit_rms((h @ t["l0.mix.dkv"].double().T)[:, :R], eps) * t["l0.mix.dkv.norm"].double()
    s = q @ (lat @ t["l0.mix.uk"].double().T)[:, :16].T
    qi, kj = divmod(int(s.argmax()), 40)
    return cfg, t, qi, kj, s


@gpu
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("dtype,tol,R", [(torch.float32, F32_TOL, 24), (torch.bfloat16, BF16_TOL, 24), (torch.bfloat16, BF16_TOL, 128)])
def test_a_key_just_inside_and_just_outside_the_window(decode, dtype, tol, R):
    size = 21
    cfg, t, qi, kj, s = peaked_latent_model(size, R)
    dull = [x for x in np.argsort(s[qi].numpy())[:12].tolist() if x != kj]                         # keys the hot query ignores
    T = 70
    cases = {"window_in": T - 1 - (size - 1), "window_out": T - 1 - size, "page_border_in": 56, "first": 0, "near": T - 2}
    outs = {}
    for name, j in cases.items():
        seq = [dull[i % len(dull)] for i in range(T)]
        seq[j], seq[T - 1] = kj, qi
        rig = Rig(cfg, tensors=t, dtype=dtype)
        rig.poison()
        if decode:
            rig.step([("r", seq[:T - 9])])
            got = torch.cat([rig.step([("r", [x])]) for x in seq[T - 9:]])[-1]
        else:
            got = rig.step([("r", seq[:30]), ("other", seq[:11])])                               # a second request beside it
            got = rig.step([("r", seq[30:])])[-1]
        want = rig.oracle(seq)[0][-1]
        assert rel_err(got, want) < tol, name
        outs[name] = want
    # the inputs do show an edge that is one token off: a seen and an unseen hot key give different logits
    assert rel_err(outs["window_in"], outs["window_out"]) > 0.05 and rel_err(outs["page_border_in"], outs["window_out"]) > 0.05
    assert rel_err(outs["first"], outs["window_out"]) < 0.05                                     # both unseen: nearly the same


def peaked_differential_model(every):
    """One differential-attention layer whose first score map is sharp and whose second is nearly flat."""
    cfg = make_cfg([dict(diff_attn(heads=2, kv=1, dim=16, vdim=16, diff=0.3, coef=0.5, every=every, scale=5.0), mlp=None)], width=32, vocab=40)
    t = tensors_for(cfg, 29)
    t["l0.canon1"] = t["l0.canon1"] * 0.02
    eps = cfg["norm"]["eps"]
    h = t["embed"].double()
    q = (O.unit_rms((h @ t["l0.mix.q"].double().T).view(40, 2, 2, 16), eps) * t["l0.mix.q.norm"].double())[:, 0, 0]
    k = (O.unit_rms((h @ t["l0.mix.k"].double().T).view(40, 1, 2, 16), eps) * t["l0.mix.k.norm"].double())[:, 0, 0]
    s = q @ k.T
    qi, kj = divmod(int(s.argmax()), 40)
    return cfg, t, qi, kj, s


@gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32_TOL), (torch.bfloat16, BF16_TOL)])
def test_a_far_key_among_hundreds(dtype, tol):
    """Plain causal attention over many pages: the hot key sits 280 tokens back, at a page's first place; the query's temperature
    has grown by then."""
    cfg, t, qi, kj, s = peaked_differential_model(every=7)
    dull = [x for x in np.argsort(s[qi].numpy())[:12].tolist() if x != kj]
    T = 300
    seq = [dull[i % len(dull)] for i in range(T)]
    seq[16], seq[T - 1] = kj, qi
    rig = Rig(cfg, tensors=t, pages=64, dtype=dtype)
    got = rig.step([("r", seq[:121])])
    got = torch.cat([got, rig.step([("r", seq[121:T - 2])]), rig.step([("r", seq[T - 2:T - 1])]), rig.step([("r", seq[T - 1:])])])
    want = rig.oracle(seq)[0]
    assert rel_err(got[-1], want[-1]) < tol and rel_err(got, want) < tol
    seq2 = list(seq)
    seq2[16] = dull[0]
    assert rel_err(rig.oracle(seq2)[0][-1], want[-1]) > 0.05
    flat = json.loads(json.dumps(cfg))
    flat["layers"][0]["mixer"]["q_temp"]["coef"] = 0.0                                            # and the temperature matters here
    assert rel_err(O.forward(flat, t, seq, torch.float64)[0][100:], want[100:]) > 0.02


@gpu
def test_the_first_tokens_of_a_sequence():
    """One, two and three tokens (fewer than the taps), in slots whose tails and pages hold another request's values."""
    for name in ("a", "b"):
        rig = Rig(SHAPES[name](), seed=19, slots=2, pages=16)
        V = rig.cfg.vocab_size
        rig.step([("old", toks(30, V, 1))])
        rig.end("old")
        for n in (1, 2, 3):
            t = toks(n + 1, V, 50 + n)
            got = torch.cat([rig.step([("new", t[:n])]), rig.step([("new", t[n:])])])
            assert rel_err(got, rig.oracle(t)[0]) < F32_TOL, (name, n)
            rig.end("new")


@gpu
def test_long_decoding_keeps_the_tails_and_the_window():
    rig = Rig(shape_b(), seed=29, pages=64)
    t = toks(260, rig.cfg.vocab_size, 8)
    want, _ = rig.oracle(t)
    rig.poison()
    got = torch.cat([rig.step([("r", t[:20])])] + [rig.step([("r", [x])]) for x in t[20:]])
    assert rel_err(got, want) < F32_TOL and rel_err(got[-1], want[-1]) < F32_TOL
    rb = Rig(shape_b(), seed=29, pages=64, dtype=torch.bfloat16)
    gb = torch.cat([rb.step([("r", t[:20])])] + [rb.step([("r", [x])]) for x in t[20:]])
    assert rel_err(gb, want) < BF16_TOL


def random_shape(seed):
    """A random configuration: layer order, head counts, sizes (multiples of eight and not), windows from one token to longer than
    the sequence, taps, constants; some layers borrow an earlier layer's weights."""
    r = random.Random(seed)
    layers = []
    for i in range(r.choice([2, 3, 4])):
        mlp = None if r.random() < 0.25 else dense(r.choice([8, 24, 40, 100]))
        same = [j for j, L in enumerate(layers) if "weights_of" not in L]
        if same and r.random() < 0.3:
            j = r.choice(same)
            layers.append(dict(json.loads(json.dumps(layers[j])), weights_of=j))
            continue
        if r.random() < 0.5:
            kv = r.choice([1, 2, 3, 4])
            layers.append(dict(diff_attn(heads=kv * r.choice([1, 2, 3, 5]), kv=kv, dim=r.choice([8, 16, 20, 24, 32, 64]), vdim=r.choice([8, 16, 32, 40, 64, 96]),
                                         diff=r.choice([0.1, 0.25, 0.5, 0.9]), coef=r.choice([0.0, 0.3, 1.0]), every=r.choice([1, 3, 16, 64]),
                                         scale=r.choice([0.1, 0.25, 0.5])), mlp=mlp))
            if r.random() < 0.2:
                layers[-1]["mixer"]["mask"] = {"size": r.choice([3, 12])}
        else:
            rd = r.choice([4, 8, 16])
            layers.append(dict(latent(heads=r.choice([1, 2, 5, 8, 16, 33]), dim=r.choice([8, 16, 24]), rot_dim=rd, vdim=r.choice([8, 16, 24]),
                                      kv_rank=r.choice([16, 32, 40, 64, 96, 128]), q_rank=r.choice([8, 24]), size=r.choice([1, 2, 5, 8, 9, 17, 40, 1000]),
                                      base=r.choice([100.0, 10000.0]), scale=r.choice([0.1, 0.25])), mlp=mlp))
    return make_cfg(layers, width=r.choice([32, 48, 64, 72, 100]), vocab=r.choice([17, 64, 131]), taps=r.choice([1, 2, 3, 4, 6]), eps=r.choice([1e-5, 1e-6]))


@gpu
@pytest.mark.parametrize("seed", range(12))
def test_random_configurations_in_a_mixed_schedule(seed):
    """Two requests cut at random into portions and single tokens, side by side from poisoned pools and tails, float32 and bfloat16."""
    cfg = random_shape(seed)
    r = random.Random(100 + seed)
    V = cfg["vocab"]
    a, b = toks(45, V, seed), toks(29, V, seed + 50)
    for dtype, tol in ((torch.float32, F32_TOL), (torch.bfloat16, 2 * BF16_TOL)):
        rig = Rig(cfg, seed=seed, dtype=dtype, pages=32)
        want_a, want_b = rig.oracle(a)[0], rig.oracle(b)[0]
        rig.poison()
        got_a, got_b, ia, ib = [], [], 0, 0
        while ia < len(a) or ib < len(b):
            na = min(len(a) - ia, r.choice([1, 1, 2, 3, 7, 16]))
            nb = min(len(b) - ib, r.choice([0, 1, 1, 2, 5, 11])) if ia > 6 else 0
            entries = ([("a", a[ia:ia + na])] if na else []) + ([("b", b[ib:ib + nb])] if nb else [])
            if not entries:
                entries, nb = [("b", b[ib:ib + 1])], 1
            out = rig.step(entries)
            got_a.append(out[:na]); got_b.append(out[na:])
            ia += na; ib += nb
        assert rel_err(torch.cat(got_a), want_a) < tol and rel_err(torch.cat(got_b), want_b) < tol, (seed, dtype, cfg)


def _write_model(tmp_path, cfg_dict, tensors):
    from safetensors.torch import save_file
    (tmp_path / "config.json").write_text(json.dumps(cfg_dict))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()}, str(tmp_path / "model.safetensors"))
    return str(tmp_path)


def _oracle_greedy(cfg_dict, tensors, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(O.forward(cfg_dict, tensors, seq, torch.float64)[0][-1].argmax()))
    return seq[len(prompt):]


@gpu
def test_greedy_generation_through_the_engine_and_its_scheduler(tmp_path):
    """LLM.generate on a checkpoint directory: registry -> loader -> scheduler (prompts cut to the token budget, admissions
    limited by two slots, pages reused) -> ragged step -> argmax.  float32 so that the greedy choice is the oracle's."""
    from jacobiforcing_amd import LLM, SamplingParams
    cfg_dict = shape_b()
    tensors = tensors_for(cfg_dict, 31)
    path = _write_model(tmp_path, cfg_dict, tensors)
    V = cfg_dict["vocab"]
    prompts = [toks(n, V, 40 + n) for n in (70, 5, 33, 1)]
    llm = LLM(path, tokenizer_path="none", dtype="float32", kvcache_block_size=64, num_kvcache_blocks=4, max_num_seqs=2, max_model_len=128,
              max_num_batched_tokens=128, device="cuda")
    out = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True), use_tqdm=False)
    for p, o in zip(prompts, out):
        assert o["token_ids"] == _oracle_greedy(cfg_dict, tensors, p, 6)
    assert len(llm.scheduler.block_manager.free_block_ids) == 4 and len(llm.model_runner.free_rows) == 2
    # the same engine replays a given schedule: portions beside single tokens, requests that end, logits where asked
    a, b = prompts[0], prompts[2]
    l1 = llm.replay_step([("a", a[:40], [0, 39]), ("b", b[:2], [])])
    l2 = llm.replay_step([("a", a[40:], [29]), ("b", b[2:], [len(b) - 3])], end=["a"])
    l3 = llm.replay_step([("c", a, [len(a) - 1])], end=["b", "c"])
    wa, wb = O.forward(cfg_dict, tensors, a, torch.float64)[0], O.forward(cfg_dict, tensors, b, torch.float64)[0]
    assert tuple(l1.shape) == (2, V) and rel_err(l1.cpu(), wa[[0, 39]]) < F32_TOL
    assert rel_err(l2.cpu(), torch.stack([wa[69], wb[len(b) - 1]])) < F32_TOL and rel_err(l3.cpu(), wa[-1:]) < F32_TOL
    assert len(llm.scheduler.block_manager.free_block_ids) == 4 and len(llm.model_runner.free_rows) == 2


@gpu
def test_sampling_through_the_engine_follows_the_distribution(tmp_path):
    from jacobiforcing_amd import LLM, SamplingParams
    cfg_dict = shape_b()
    tensors = tensors_for(cfg_dict, 37)
    path = _write_model(tmp_path, cfg_dict, tensors)
    prompt = toks(9, cfg_dict["vocab"], 50)
    llm = LLM(path, tokenizer_path="none", dtype="float32", kvcache_block_size=64, num_kvcache_blocks=16, max_num_seqs=16, max_model_len=64,
              max_num_batched_tokens=64, device="cuda")
    torch.manual_seed(0)
    out = llm.generate([prompt] * 800, SamplingParams(temperature=1.0, max_tokens=1, ignore_eos=True), use_tqdm=False)
    p = torch.softmax(O.forward(cfg_dict, tensors, prompt, torch.float64)[0][-1], 0).numpy()
    counts = np.bincount([o["token_ids"][0] for o in out], minlength=len(p)) / 800.0
    assert 0.5 * np.abs(counts - p).sum() < 0.2                                                 # total variation of 800 draws over 77 ids
