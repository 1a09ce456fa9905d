"""Lokizen through the package (HIP layer kernels, paged pool + state slots, ragged step, scheduler, LLM.generate) against the
plain oracle ``oracle/lokizen_oracle.py``, which shares no code with it.  Small random models of several shapes; where random
weights would hide a fault (a key at a window's edge among many) the inputs are chosen so that one score stands out.

CPU tests cover the oracle's own pieces, the config reader, the bucket table and the page / slot bookkeeping; everything that
launches a kernel is marked ``gpu``."""
import json
import math
import random

import numpy as np
import pytest
import torch

from oracle import lokizen_oracle as O
from jacobiforcing_amd.modeling import MODEL_REGISTRY, read_model_config
from jacobiforcing_amd.modeling import lokizen as LK

gpu = pytest.mark.gpu


# ---- model shapes -----------------------------------------------------------------------------------------------------------------
def attn(heads=6, kv=2, dim=24, vdim=40, size=12, keep=3, bias_max=40, scale=0.3):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "bias_max": bias_max,
                                           "mask": {"size": size, "keep_first": keep}}}


def ret(heads=3, dim=24, vdim=40, dims=16, base=500.0, decay=None):
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "rot": {"dims": dims, "base": base},
                                           "decay": decay or [1 - 2.0 ** (-3 - h) for h in range(heads)]}}


def moe(experts=5, top=2, ff=56, scale=1.25):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale}}


def make_cfg(layers, width=96, vocab=131, loop=None, eps=1e-5, emb=0.75):
    d = {"architecture": "Lokizen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": emb}, "layers": layers}
    if loop:
        d["loop"] = loop
    return d


def shape_a():
    """Looped span in the middle, a layer without feed-forward, grouped key/value heads, partial rotation."""
    return make_cfg([dict(ret(), mlp=moe()), dict(attn(), mlp=moe()), dict(ret(heads=2, dim=40, vdim=24, dims=40), mlp=None),
                     dict(attn(heads=4, kv=4, dim=16, vdim=16, size=7, keep=0, bias_max=20), mlp=moe(experts=3, top=3, ff=40))],
                    loop={"start": 1, "stop": 3, "times": 2})


def shape_b():
    """No loop, one head, every expert chosen, a window of one page and more kept tokens than window."""
    return make_cfg([dict(attn(heads=1, kv=1, dim=32, vdim=72, size=8, keep=10, bias_max=64), mlp=moe(experts=2, top=2, ff=24)),
                     dict(ret(heads=1, dim=64, vdim=130, dims=64, base=10000.0, decay=[0.96875]), mlp=moe(experts=9, top=1, ff=33, scale=1.0))],
                    width=64, vocab=77, emb=1.0, eps=1e-6)


SHAPES = {"a": shape_a, "b": shape_b}


def tensors_for(cfg_dict, seed, rel_rows=10):
    return LK.random_tensors(LK.LokizenConfig.from_dict(cfg_dict), seed, rel_rows=rel_rows)


def oracle_logits(cfg_dict, tensors, tokens):
    return O.forward(cfg_dict, tensors, tokens, torch.float64)


def rel_err(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    return float(np.sqrt(((got - want) ** 2).mean()) / max(np.sqrt((want ** 2).mean()), 1e-30))


F32_TOL, BF16_TOL = 2e-4, 6e-2


def close(got, want, tol):
    """float32: the whole tensor within ``tol``.  bfloat16 (tol = BF16_TOL): the typical token within ``tol`` — a router score
    that bfloat16 rounds across a near tie picks another expert for that token (and, through a recurrent state, colours a few
    tokens behind it), which is rounding, not a fault; the float32 comparisons are the sharp ones."""
    if tol < 1e-2:
        return rel_err(got, want) < tol
    per = [rel_err(got[i], want[i]) for i in range(len(want))]
    return float(np.median(per)) < tol


# =====================================================================================================================================
# CPU: oracle pieces, config reader, tables, bookkeeping
# =====================================================================================================================================
def test_registry_reads_the_architecture_key(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(shape_a()))
    cfg = read_model_config(tmp_path)
    assert isinstance(cfg, LK.LokizenConfig) and cfg.family == "ragged" and "Lokizen" in MODEL_REGISTRY
    assert cfg.vocab_size == 131 and cfg.hidden_size == 96 and cfg.num_hidden_layers == 4
    (tmp_path / "config.json").write_text(json.dumps({"architecture": "Nonesuch"}))
    with pytest.raises(ValueError):
        read_model_config(tmp_path)


def test_layer_runs_follow_the_loop():
    cfg = LK.LokizenConfig.from_dict(shape_a())
    assert cfg.runs() == [(0, False), (1, False), (2, False), (1, True), (2, False), (3, False)] == O.layer_runs(shape_a())
    plain = LK.LokizenConfig.from_dict(shape_b())
    assert plain.runs() == [(0, False), (1, False)] == O.layer_runs(shape_b())
    whole = make_cfg([dict(ret(), mlp=None)] * 3, loop={"start": 0, "stop": 3, "times": 3})
    r = LK.LokizenConfig.from_dict(whole).runs()
    assert len(r) == 9 and [x for _, x in r] == [False] * 3 + [True, False, False] * 2 and r == O.layer_runs(whole)
    with pytest.raises(ValueError):
        LK.LokizenConfig.from_dict(make_cfg([dict(ret(), mlp=None)], loop={"start": 1, "stop": 0, "times": 2}))


@pytest.mark.parametrize("rows,far", [(16, 240), (10, 40), (8, 64), (32, 128), (7, 19)])
def test_distance_bucket_table_matches_the_scalar_rule(rows, far):
    lut = LK.distance_bucket_table(rows, far, 600)
    assert lut.tolist() == [O.distance_bucket(n, rows, far) for n in range(600)]
    assert lut[0] == 0 and lut.max() == rows - 1 and (np.diff(lut) >= 0).all() and lut[rows // 2 - 1] == rows // 2 - 1


def test_oracle_mask_and_rotation():
    assert O.visible(20, 20, 4, 2) and O.visible(20, 17, 4, 2) and not O.visible(20, 16, 4, 2) and O.visible(20, 1, 4, 2)
    assert not O.visible(20, 2, 4, 2) and not O.visible(3, 4, 4, 2)
    x = torch.randn(5, 2, 12, dtype=torch.float64)
    y = O.rotate_half_pairs(x, 8, 100.0)
    assert torch.equal(y[..., 8:], x[..., 8:]) and torch.allclose(y[0], x[0])                       # position 0: no rotation
    assert torch.allclose((y[..., :8] ** 2).sum(-1), (x[..., :8] ** 2).sum(-1))                     # a rotation keeps the length
    # scores of rotated q, k depend on the distance only
    q, k = torch.randn(1, 1, 8, dtype=torch.float64), torch.randn(1, 1, 8, dtype=torch.float64)
    rq, rk = O.rotate_half_pairs(q.expand(9, 1, 8), 8, 100.0), O.rotate_half_pairs(k.expand(9, 1, 8), 8, 100.0)
    assert abs(float((rq[7] * rk[4]).sum() - (rq[5] * rk[2]).sum())) < 1e-5          # the angles are float32


def test_oracle_retention_equals_its_unrolled_sum():
    torch.manual_seed(0)
    m = ret(heads=2, dim=8, vdim=6, dims=0)["mixer"]
    T, W = 9, 16
    P = {"mix.q": torch.randn(16, W, dtype=torch.float64), "mix.k": torch.randn(16, W, dtype=torch.float64), "mix.v": torch.randn(12, W, dtype=torch.float64),
         "mix.g": torch.randn(12, W, dtype=torch.float64), "mix.o": torch.eye(12, dtype=torch.float64)}
    h = torch.randn(T, W, dtype=torch.float64)
    got = O.retention_mixer(h, P, m, 1e-5)
    q, k, v = (h @ P["mix.q"].T).view(T, 2, 8), (h @ P["mix.k"].T).view(T, 2, 8) * 8 ** -0.5, (h @ P["mix.v"].T).view(T, 2, 6)
    g = h @ P["mix.g"].T
    for t in (0, 4, 8):
        o = torch.stack([sum(m["decay"][hh] ** (t - s) * (q[t, hh] @ k[s, hh]) * v[s, hh] for s in range(t + 1)) for hh in range(2)])
        o = (o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-5)).reshape(-1) * (g[t] * torch.sigmoid(g[t]))
        assert torch.allclose(got[t], o, atol=1e-10)


def test_oracle_router_uses_correction_for_choice_only():
    W = 8
    h = torch.ones(1, W, dtype=torch.float64)
    P = {"mlp.router": torch.zeros(3, W, dtype=torch.float64), "mlp.correction": torch.tensor([0.0, 5.0, -5.0], dtype=torch.float64)}
    P["mlp.router"][2] = 1.0                                   # expert 2 has the largest score, expert 1 the largest choice score
    for e in range(3):
        P[f"mlp.e{e}.up"] = torch.eye(W, dtype=torch.float64) * (e + 1)
        P[f"mlp.e{e}.down"] = torch.eye(W, dtype=torch.float64)
    out = O.moe_feed_forward(h, P, moe(experts=3, top=1, scale=2.0))
    assert torch.allclose(out, torch.full((1, W), 0.5 * 2.0 * 4.0, dtype=torch.float64))   # sigmoid(0) * scale * relu(2)^2: no correction in the weight


def test_pages_are_allocated_per_token_count_and_reused():
    from jacobiforcing_amd.engine.block_manager import BlockManager
    from jacobiforcing_amd.engine.sequence import Sequence
    bm = BlockManager(5, 64)
    a, b = Sequence(list(range(130))), Sequence(list(range(10)))
    assert bm.ensure(a, 64) and a.block_table == [0] and bm.ensure(a, 65) and a.block_table == [0, 1]
    assert bm.ensure(a, 65) and len(a.block_table) == 2                                      # nothing more for the same count
    assert bm.ensure(b, 10) and b.block_table == [2]
    assert not bm.ensure(a, 64 * 5) and len(a.block_table) == 2                              # all or nothing
    bm.deallocate(b)
    assert bm.ensure(a, 64 * 4)                                                              # b's page went to the END of the free list
    assert set(a.block_table) == {0, 1, 3, 4} and len(bm.free_block_ids) == 1 and bm.free_block_ids[0] == 2


def _cpu_scheduler(tmp_path, **kw):
    from jacobiforcing_amd.config import Config
    from jacobiforcing_amd.engine.scheduler import Scheduler
    (tmp_path / "config.json").write_text(json.dumps(shape_b()))
    cfg = Config(str(tmp_path), kvcache_block_size=64, **kw)
    cfg.eos = -1
    return Scheduler(cfg)


def test_ragged_schedule_mixes_portions_and_single_tokens(tmp_path):
    from jacobiforcing_amd.engine.sequence import Sequence
    from jacobiforcing_amd.sampling_params import SamplingParams
    sch = _cpu_scheduler(tmp_path, num_kvcache_blocks=8, max_num_seqs=4, max_model_len=256, max_num_batched_tokens=256)
    sch.row_capacity = 2
    sp = SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True)
    s1, s2, s3 = Sequence(list(range(300 % 77, 300 % 77 + 200)), sp), Sequence([1, 2, 3], sp), Sequence([4, 5], sp)
    for s in (s1, s2, s3):
        sch.add(s)
    items = sch.schedule_ragged()
    assert [(s.seq_id, n) for s, n in items] == [(s1.seq_id, 200), (s2.seq_id, 3)]              # two slots: s3 waits
    for s, n in items:
        s.num_cached_tokens += n
    sch.postprocess([s1, s2], [7, 8])
    items = sch.schedule_ragged()
    assert [(s.seq_id, n) for s, n in items] == [(s1.seq_id, 1), (s2.seq_id, 1)]
    for s, n in items:
        s.num_cached_tokens += n
    sch.finish(s2)
    sch.postprocess([s1], [9])
    items = sch.schedule_ragged()                                                              # a decoded token beside a new prompt
    assert [(s.seq_id, n) for s, n in items] == [(s1.seq_id, 1), (s3.seq_id, 2)]
    assert set(s3.block_table) & set(s1.block_table) == set()


def test_ragged_schedule_cuts_a_prompt_to_the_token_budget(tmp_path):
    from jacobiforcing_amd.engine.sequence import Sequence
    sch = _cpu_scheduler(tmp_path, num_kvcache_blocks=8, max_num_seqs=4, max_model_len=100, max_num_batched_tokens=100)
    s = Sequence(list(range(70)) * 3)
    sch.add(s)
    seen = []
    while s.num_cached_tokens < len(s):
        (q, n), = sch.schedule_ragged()
        seen.append(n)
        q.num_cached_tokens += n
    assert seen == [100, 100, 10] and len(s.block_table) == 4


def test_config_rejects_small_pages_for_padded_families_only(tmp_path):
    from jacobiforcing_amd.config import Config
    (tmp_path / "config.json").write_text(json.dumps(shape_b()))
    assert Config(str(tmp_path), kvcache_block_size=64, dtype="float32").dtype == "float32"
    with pytest.raises(AssertionError):
        Config(str(tmp_path), kvcache_block_size=100)
    with pytest.raises(ValueError):
        Config(str(tmp_path), kvcache_block_size=64, dtype="float16")


# =====================================================================================================================================
# GPU: the package against the oracle
# =====================================================================================================================================
class Rig:
    """A model on the GPU with a pool of shuffled pages; runs steps of (request, tokens) and keeps the bookkeeping a test needs."""

    def __init__(self, cfg_dict, seed=0, dtype=torch.float32, page=8, pages=64, slots=4, rel_rows=10, tensors=None):
        from jacobiforcing_amd import layer_ops as LO
        self.LO = LO
        self.cfg_dict = cfg_dict
        self.cfg = LK.LokizenConfig.from_dict(cfg_dict)
        self.tensors = tensors or tensors_for(cfg_dict, seed, rel_rows)
        self.model = LK.LokizenModel(self.cfg, LK.LokizenWeights(self.cfg, self.tensors, "cuda", dtype), max_positions=1024)
        self.page = page
        self.cache = self.model.new_cache(pages, page, slots)
        self.free_pages = list(range(pages))
        random.Random(seed).shuffle(self.free_pages)
        self.free_slots = list(range(slots))[::-1]
        self.req = {}

    def poison(self):
        """Fill pool and state with large values: whatever a kernel reads without having written it shows."""
        for t in self.cache.k + self.cache.v + self.cache.state:
            if t is not None:
                t.fill_(1e4)

    def step(self, entries, trace=None):
        """entries = [(key, tokens)]; returns logits [sum of tokens, vocab] (float, on the CPU)."""
        counts, starts, slots, tables, ids = [], [], [], [], []
        for key, toks in entries:
            r = self.req.setdefault(key, {"n": 0, "pages": [], "slot": None})
            if r["slot"] is None:
                r["slot"] = self.free_slots.pop()
            while len(r["pages"]) * self.page < r["n"] + len(toks):
                r["pages"].append(self.free_pages.pop())
            counts.append(len(toks)); starts.append(r["n"]); slots.append(r["slot"]); tables.append(r["pages"])
            ids += list(toks)
            r["n"] += len(toks)
        b = self.LO.RaggedBatch.build(counts, starts, slots, tables, self.page, "cuda")
        return self.model.forward(torch.tensor(ids, device="cuda"), b, self.cache, None, trace).cpu()

    def end(self, key):
        r = self.req.pop(key)
        self.free_pages += r["pages"][::-1]
        self.free_slots.append(r["slot"])

    def oracle(self, tokens):
        return O.forward(self.cfg_dict, self.tensors, list(tokens), torch.float64)


def toks(n, vocab, seed):
    return [random.Random(seed * 7919 + i).randrange(vocab) for i in range(n)]


@gpu
@pytest.mark.parametrize("W,count", [(96, 1), (200, 3), (1000, 2)])
def test_residual_update_and_norm(W, count):
    from jacobiforcing_amd import layer_ops as LO
    g = torch.Generator().manual_seed(W)
    x, y, x0, w = torch.randn(5, W, generator=g), torch.randn(5, count, W, generator=g), torch.randn(5, W, generator=g), torch.randn(W, generator=g)
    want_x = x.double() + y.double().sum(1) + x0.double()
    want = O.rms_norm(want_x, w.double(), 1e-5)
    xd = x.cuda()
    out = LO.add_rmsnorm(xd, y.cuda(), x0.cuda(), w.cuda(), 1e-5, torch.float32)
    assert rel_err(xd.cpu(), want_x) < 1e-6 and rel_err(out.cpu(), want) < 1e-6
    xb = x.cuda()
    outb = LO.add_rmsnorm(xb, y.cuda().bfloat16(), None, w.cuda().bfloat16(), 1e-5, torch.bfloat16)
    wantb = O.rms_norm(x.double() + y.bfloat16().double().sum(1), w.bfloat16().double(), 1e-5)
    assert xb.dtype == torch.float32 and rel_err(outb.float().cpu(), wantb) < 6e-3
    assert LO.add_rmsnorm(xd, None, None, None, 1e-5, None) is None                              # nothing to add, nothing to norm
    tiny = torch.full((1, W), 1e-4).cuda()                                                     # eps inside the root decides here
    assert rel_err(LO.add_rmsnorm(tiny, None, None, None, 1e-5, torch.float32).cpu(), O.rms_norm(torch.full((1, W), 1e-4).double(), None, 1e-5)) < 1e-6


@gpu
@pytest.mark.parametrize("name", ["a", "b"])
def test_each_mixer_and_feed_forward_alone(name):
    """Layer by layer on the oracle's own inputs: mixer output and expert output for a whole prompt."""
    import torch.nn.functional as F
    rig = Rig(SHAPES[name](), seed=3)
    T = 37
    g = torch.Generator().manual_seed(1)
    h = torch.randn(T, rig.cfg.hidden_size, generator=g)
    b = rig.LO.RaggedBatch.build([T], [0], [1], [[9, 3, 20, 11, 5]], 8, "cuda")
    for run, (li, _) in enumerate(rig.model.runs):
        L, P = rig.cfg_dict["layers"][li], {k: v.double() for k, v in O.layer_tensors(rig.tensors, li).items()}
        lw = rig.model.w.layers[li]
        if L["type"] == "attention":
            got, want = rig.model._attention(run, li, h.cuda(), b, rig.cache), O.attention_mixer(h.double(), P, L["mixer"], rig.cfg.norm_eps)
        else:
            got, want = rig.model._retention(run, li, h.cuda(), b, rig.cache), O.retention_mixer(h.double(), P, L["mixer"], rig.cfg.norm_eps)
        assert rel_err(F.linear(got, lw["w_o"]).cpu(), want) < 1e-5, (li, L["type"])
        if L.get("mlp"):
            r = L["mlp"]["router"]
            y = rig.LO.moe_experts(h.cuda(), F.linear(h.cuda(), lw["router"]), lw["correction"], r["top"], r["scale"], lw["w_up"], lw["w_down"])
            assert tuple(y.shape) == (T, r["top"], rig.cfg.hidden_size)
            assert rel_err(y.sum(1).cpu(), O.moe_feed_forward(h.double(), P, L["mlp"])) < 1e-5, li


@gpu
@pytest.mark.parametrize("name", ["a", "b"])
def test_whole_prompt_and_every_layer_run(name):
    rig = Rig(SHAPES[name](), seed=5)
    t = toks(61, rig.cfg.vocab_size, 1)
    trace = []
    got = rig.step([("p", t)], trace)
    want, want_trace = rig.oracle(t)
    assert len(trace) == want_trace.shape[0]
    for i, x in enumerate(trace):
        assert rel_err(x.cpu(), want_trace[i]) < 1e-5, f"layer run {i}"
    assert rel_err(got, want) < F32_TOL
    assert close(Rig(SHAPES[name](), seed=5, dtype=torch.bfloat16).step([("p", t)]), want, BF16_TOL)


@gpu
@pytest.mark.parametrize("name", ["a", "b"])
def test_prefill_equals_token_by_token_decoding(name):
    """The first tokens of a sequence, a window passing over decoded tokens, state carried from token to token."""
    rig = Rig(SHAPES[name](), seed=7)
    t = toks(45, rig.cfg.vocab_size, 2)
    want, _ = rig.oracle(t)
    rig.poison()
    one = torch.cat([rig.step([("d", [x])]) for x in t])
    assert rel_err(one, want) < F32_TOL
    for i in (0, 1, 2, 9, 44):
        assert rel_err(one[i], want[i]) < F32_TOL, i
    rig.poison()
    assert rel_err(rig.step([("w", t)]), want) < F32_TOL


@gpu
@pytest.mark.parametrize("cuts", [[2] * 20, [1, 2, 3, 5, 8, 13, 7, 1], [7, 9, 8, 16], [39, 1], [3, 37]])
def test_portions_of_any_size(cuts):
    """Portions cut in the middle of pages (8 tokens) and windows (12 and 7 tokens), down to two tokens."""
    rig = Rig(shape_a(), seed=11)
    t = toks(sum(cuts), rig.cfg.vocab_size, 3)
    want, _ = rig.oracle(t)
    rig.poison()
    out, o = [], 0
    for c in cuts:
        out.append(rig.step([("c", t[o:o + c])]))
        o += c
    got = torch.cat(out)
    assert rel_err(got, want) < F32_TOL
    worst = max(rel_err(got[i], want[i]) for i in range(len(t)))
    assert worst < 5 * F32_TOL, worst


@gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32_TOL), (torch.bfloat16, BF16_TOL)])
def test_long_portions_run_in_chunks(dtype, tol):
    """Portions of two chunks and more take the recurrent layers' chunked launches (local states, join, outputs): from position 0
    and from a carried state, a last chunk that is short, beside a request that is scanned in one piece; then decoding goes on
    from the joined state."""
    from jacobiforcing_amd import layer_ops as LO
    rig = Rig(shape_a(), seed=41, pages=96, dtype=dtype)
    V, C = rig.cfg.vocab_size, LO.RETENTION_CHUNK
    a, b = toks(2 * C + 90, V, 9), toks(3 * C + 5, V, 10)
    wa, wb = rig.oracle(a)[0], rig.oracle(b)[0]
    rig.poison()
    g1 = rig.step([("a", a[:2 * C + 17]), ("b", b[:11])])                       # a: three chunks (the last of 17), b: one scan
    g2 = rig.step([("a", a[2 * C + 17:2 * C + 18]), ("b", b[11:11 + 2 * C])])    # b: two full chunks from a carried state
    g3 = rig.step([("a", a[2 * C + 18:]), ("b", b[11 + 2 * C:])])
    na = 2 * C + 17
    got_a = torch.cat([g1[:na], g2[:1], g3[:len(a) - na - 1]])
    got_b = torch.cat([g1[na:], g2[1:], g3[len(a) - na - 1:]])
    assert close(got_a, wa, tol) and close(got_b, wb, tol)
    if dtype == torch.float32:
        assert rel_err(got_a[-1], wa[-1]) < 3 * tol and rel_err(got_b[-1], wb[-1]) < 3 * tol


@gpu
@pytest.mark.parametrize("H,G,D,Dv,direct", [(12, 4, 64, 128, True), (8, 2, 128, 64, True), (3, 1, 24, 40, False), (16, 16, 32, 32, True),
                                               (5, 5, 8, 100, True), (20, 4, 16, 24, True), (4, 2, 12, 20, False)])
def test_bfloat16_attention_alone(H, G, D, Dv, direct, monkeypatch):
    """bfloat16 attention alone on bfloat16-rounded inputs: the MFMA kernel (one or two heads per wavefront, value widths that are
    no multiple of its 32-column tiles) and, for more than 16 heads or a head size that is no multiple of 8, the float-FMA kernel;
    the bias by distance directly or through the bucket table.  Two portions that cut a window, then single tokens, pages out of
    order."""
    import torch.nn.functional as F
    if not direct:
        monkeypatch.setattr(LK, "DIRECT_BIAS_POSITIONS", 0)
    cfg = make_cfg([dict(attn(heads=H, kv=G, dim=D, vdim=Dv, size=37, keep=5, bias_max=90, scale=D ** -0.5), mlp=None)], width=64, vocab=50)
    rig = Rig(cfg, seed=H, dtype=torch.bfloat16, pages=32)
    T = 110
    g = torch.Generator().manual_seed(H + D)
    h = torch.randn(T, 64, generator=g).bfloat16()
    P = {k: v.double() for k, v in O.layer_tensors(rig.tensors, 0).items()}
    want = O.attention_mixer(h.double(), P, cfg["layers"][0]["mixer"], rig.cfg.norm_eps)
    pages = list(range(31, 31 - 14, -1))
    rig.poison()
    got, at = [], 0
    for n in (70, 37, 1, 1, 1):
        b = rig.LO.RaggedBatch.build([n], [at], [0], [pages], 8, "cuda")
        got.append(F.linear(rig.model._attention(0, 0, h[at:at + n].cuda(), b, rig.cache), rig.model.w.layers[0]["w_o"]).float().cpu())
        at += n
    got = torch.cat(got)
    assert rel_err(got, want) < 2e-2
    assert max(rel_err(got[i], want[i]) for i in range(T)) < 6e-2


@gpu
def test_grouped_expert_products_on_the_matrix_cores():
    """bfloat16 with a depth that is a multiple of 8 takes the MFMA kernel: many rows per expert, experts without rows, row counts
    that are no multiple of the tile, output widths that are no multiple of 128."""
    from jacobiforcing_amd import layer_ops as LO
    g = torch.Generator().manual_seed(4)
    n, E, top, W, ff = 300, 6, 2, 72, 200
    z = torch.randn(n, E, generator=g)
    z[:, 4] = -30.0                                                             # nobody chooses expert 4
    h = torch.randn(n, W, generator=g).bfloat16()
    up, down = (torch.randn(E, ff, W, generator=g) * W ** -0.5).bfloat16(), (torch.randn(E, W, ff, generator=g) * ff ** -0.5).bfloat16()
    y = LO.moe_experts(h.cuda(), z.cuda(), None, top, 1.5, up.cuda(), down.cuda()).cpu().double().sum(1)
    s = torch.sigmoid(z.double())
    want = torch.zeros(n, W, dtype=torch.float64)
    for i in range(n):
        for e in torch.topk(s[i], top).indices.tolist():
            act = (torch.relu(up[e].double() @ h[i].double()) ** 2).bfloat16().double()           # the activations are stored in bfloat16
            want[i] += s[i, e] * 1.5 * (down[e].double() @ act)
    assert rel_err(y, want) < 2e-3


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
def test_freed_pages_and_slots_are_used_again():
    """Four slots, a pool that holds two requests: requests end, their pages and slots go to new ones, old content must not leak."""
    rig = Rig(shape_a(), seed=17, pages=12, slots=2)
    V = rig.cfg.vocab_size
    rig.poison()
    for rnd in range(4):
        a, b = toks(40 + rnd, V, 20 + rnd), toks(17 + 3 * rnd, V, 30 + rnd)
        ga = rig.step([("a", a[:25]), ("b", b[:5])])
        gb = rig.step([("a", a[25:]), ("b", b[5:])])
        got_a = torch.cat([ga[:25], gb[:len(a) - 25]])
        got_b = torch.cat([ga[25:], gb[len(a) - 25:]])
        assert rel_err(got_a, rig.oracle(a)[0]) < F32_TOL and rel_err(got_b, rig.oracle(b)[0]) < F32_TOL, rnd
        used = set(rig.req["a"]["pages"]) | set(rig.req["b"]["pages"])
        rig.end("b"); rig.end("a")
        assert len(rig.free_pages) == 12 and len(used) >= 8


def peaked_attention_model(size, keep, rel_rows=8, bias_max=32):
    """One attention layer, no feed-forward, a sharp softmax.  Returns (cfg, tensors, hot query token, hot key token): the
    pair of tokens whose score is the largest among all pairs, by a wide margin after the model's scale."""
    cfg = make_cfg([dict(attn(heads=2, kv=1, dim=16, vdim=16, size=size, keep=keep, bias_max=bias_max, scale=6.0), mlp=None)], width=32, vocab=40)
    t = tensors_for(cfg, 23, rel_rows)
    t["l0.mix.rel"] = t["l0.mix.rel"] * 0.1
    eps = cfg["norm"]["eps"]
    h = O.rms_norm(t["embed"].double() * cfg["embedding"]["scale"], t["l0.norm1"].double(), eps)
    q = O.rms_norm(h @ t["l0.mix.q"].double().T, t["l0.mix.q.norm"].double(), eps)[:, :16]
    k = O.rms_norm(h @ t["l0.mix.k"].double().T, t["l0.mix.k.norm"].double(), eps)
    s = q @ k.T
    qi, kj = divmod(int(s.argmax()), 40)
    return cfg, t, qi, kj, s


@gpu
@pytest.mark.parametrize("decode", [False, True])
def test_a_key_just_inside_and_just_outside_the_window_and_the_kept_tokens(decode):
    size, keep = 21, 5
    cfg, t, qi, kj, s = peaked_attention_model(size, keep)
    dull = [x for x in np.argsort(s[qi].numpy())[:12].tolist() if x != kj]                         # keys the hot query ignores
    T = 70
    cases = {"window_in": T - 1 - (size - 1), "window_out": T - 1 - size, "first_in": keep - 1, "first_out": keep, "far_page_border": 8,
             "near": T - 2}
    outs = {}
    for name, j in cases.items():
        seq = [dull[i % len(dull)] for i in range(T)]
        seq[j], seq[T - 1] = kj, qi
        rig = Rig(cfg, tensors=t)
        rig.poison()
        if decode:
            rig.step([("r", seq[:T - 9])])
            got = torch.cat([rig.step([("r", [x])]) for x in seq[T - 9:]])[-1]
        else:
            got = rig.step([("r", seq[:30]), ("other", seq[:11])])                               # a second request beside it
            got = rig.step([("r", seq[30:])])[-1]
        want = rig.oracle(seq)[0][-1]
        assert rel_err(got, want) < F32_TOL, name
        outs[name] = want
    # the inputs do show an edge that is one token off: seen and unseen hot keys give different logits
    assert rel_err(outs["window_in"], outs["window_out"]) > 0.05 and rel_err(outs["first_in"], outs["first_out"]) > 0.05
    assert rel_err(outs["far_page_border"], outs["first_out"]) < 0.05                             # both unseen: nearly the same


@gpu
def test_a_far_key_among_hundreds_without_a_window():
    """A window larger than the sequence: plain causal attention over many pages; the hot key sits 180 tokens back."""
    cfg, t, qi, kj, s = peaked_attention_model(size=100000, keep=0, rel_rows=12, bias_max=500)
    dull = [x for x in np.argsort(s[qi].numpy())[:12].tolist() if x != kj]
    T = 200
    seq = [dull[i % len(dull)] for i in range(T)]
    seq[17], seq[T - 1] = kj, qi
    rig = Rig(cfg, tensors=t, pages=64, rel_rows=12)
    got = rig.step([("r", seq[:121])])
    got = torch.cat([got, rig.step([("r", seq[121:])])])
    want = rig.oracle(seq)[0]
    assert rel_err(got[-1], want[-1]) < F32_TOL and rel_err(got, want) < F32_TOL
    seq2 = list(seq)
    seq2[17] = dull[0]
    assert rel_err(rig.oracle(seq2)[0][-1], want[-1]) > 0.05


@gpu
def test_long_decoding_keeps_the_state_and_the_window():
    rig = Rig(shape_b(), seed=29, pages=64)
    t = toks(260, rig.cfg.vocab_size, 8)
    want, _ = rig.oracle(t)
    rig.poison()
    got = torch.cat([rig.step([("r", t[:20])])] + [rig.step([("r", [x])]) for x in t[20:]])
    assert rel_err(got, want) < F32_TOL and rel_err(got[-1], want[-1]) < F32_TOL
    rb = Rig(shape_b(), seed=29, pages=64, dtype=torch.bfloat16)
    gb = torch.cat([rb.step([("r", t[:20])])] + [rb.step([("r", [x])]) for x in t[20:]])
    assert close(gb, want, BF16_TOL)


@gpu
def test_router_choice_on_the_device_matches_the_rule():
    from jacobiforcing_amd import layer_ops as LO
    g = torch.Generator().manual_seed(2)
    n, E, top, W, ff = 50, 7, 3, 16, 8
    z, corr = torch.randn(n, E, generator=g) * 2, torch.randn(E, generator=g)
    h = torch.randn(n, W, generator=g)
    up, down = torch.randn(E, ff, W, generator=g), torch.randn(E, W, ff, generator=g)
    y = LO.moe_experts(h.cuda(), z.cuda(), corr.cuda(), top, 0.5, up.cuda(), down.cuda()).cpu().double()
    s = torch.sigmoid(z.double())
    for i in range(n):
        chosen = torch.topk(s[i] + corr.double(), top).indices.tolist()
        want = torch.stack([s[i, e] * 0.5 * (down[e].double() @ torch.relu(up[e].double() @ h[i].double()) ** 2) for e in chosen])
        assert torch.allclose(y[i], want, rtol=1e-4, atol=1e-4), i                                 # in the order of the choice


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
