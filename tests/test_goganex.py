"""Goganex through the engine (model registry, grouped K/V cache, state slots, Engine.step,
generation) against the plain float64 statement in ``oracle_goganex.py``, on small random
checkpoints of several shapes. Every case runs on the CPU (PyTorch statements of the ops) and,
marked ``gpu``, on the HIP kernels in fp32 and bf16.
"""
import json
import math
import os

import pytest
import torch
from safetensors.torch import save_file

import oracle_goganex as O
from theroundtaible_amd.engine import Engine, EngineConfig, SamplingParams, Turn
from theroundtaible_amd.engine.kv_cache import KVCacheOOM
from theroundtaible_amd.models.config import ParallelSpec, config_from_dir, get_config
from theroundtaible_amd.models.weights import layout_for

GPU = pytest.mark.gpu
RUNS = [("cpu", "fp32"), pytest.param(("cuda:0", "fp32"), marks=GPU), pytest.param(("cuda:0", "bf16"), marks=GPU)]
SCALING = {"factor": 4.0, "low": 1.0, "high": 3.0, "original": 48}


def att(heads, kv, dim, vdim=None, base=800.0, rot_dims=None, scaling=SCALING, scale=None, ff=56, limit=1.2):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim if vdim is None else vdim,
                      "rot": {"base": base, "dims": dim if rot_dims is None else rot_dims, "scaling": scaling},
                      "scale": 1.3 * dim ** -0.5 if scale is None else scale},
            "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


def par(heads, kv, dim, width, scale=None, ff=56, limit=1.2):
    return {"type": "parallel",
            "mixer": {"left": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim,
                               "scale": dim ** -0.5 if scale is None else scale},
                      "right": {"width": width}},
            "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


def make_config(width=40, vocab=97, layers=None, loop=(1, 3, 2), embed_scale=0.7, eps=1e-5):
    if layers is None:
        layers = [att(6, 2, 12), att(4, 4, 10, vdim=14, rot_dims=6, ff=0), par(6, 3, 8, 52)]
    cfg = {"architecture": "Goganex", "embedding": {"scale": embed_scale}, "layers": layers, "norm": {"eps": eps},
           "vocab": vocab, "width": width}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_checkpoint(path, cfg, seed=0, edit=None):
    """Random weights for ``cfg`` (a config.json dict) written as a checkpoint directory; returns
    the float64 tensors. ``edit(P)`` may change tensors before they are written."""
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    mc = config_from_dir(path)
    g = torch.Generator().manual_seed(seed)
    P = {}
    for name, (shape, _, _) in layout_for(mc).items():
        if name.endswith(("norm1", "norm2", "final.norm", ".out")):
            w = 0.6 + torch.rand(shape, generator=g)
        elif name.endswith("shift"):
            w = torch.rand(shape, generator=g)
        elif name.endswith("temp"):
            w = 0.5 + 1.5 * torch.rand(shape, generator=g)
        elif name.endswith(".b"):
            w = torch.randn(shape, generator=g) * 0.5
        elif name == "embed":
            w = torch.randn(shape, generator=g)
        else:
            w = torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        P[name] = w.to(torch.bfloat16).float()      # values both number formats hold exactly
    if edit is not None:
        edit(P)
    save_file({k: v.contiguous() for k, v in P.items()}, os.path.join(path, "model.safetensors"))
    return {k: v.double() for k, v in P.items()}


def engine_for(path, run, tokens=512, block_size=16, slots=4, graphs=False):
    device, dtype = run
    if device != "cpu":
        from theroundtaible_amd.ops import hybrid
        hybrid.native()     # the GPU cases fail loudly when the extension is missing
    return Engine(EngineConfig(model=str(path), weights=str(path), dtype=dtype, device=device, block_size=block_size,
                               num_blocks=(tokens + block_size - 1) // block_size + (1 if graphs else 0),
                               use_graphs=graphs, state_slots=slots, max_batch=slots))


def close(got, want, run, what=""):
    tol = dict(rtol=0, atol=0.3) if run[1] == "bf16" else dict(rtol=0, atol=2e-3)
    torch.testing.assert_close(got.double().cpu(), want, msg=lambda m: f"{what}: {m}", **tol)


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


# ---- each mechanism alone (package ops on the CPU against the oracle's functions) ---------------

def _one_span(T, start=0):
    """Metadata of one span of T rows at positions start .. of a sequence in slot 0."""
    return (torch.zeros(T, dtype=torch.int32), torch.arange(start, start + T), torch.tensor([start], dtype=torch.int32),
            torch.zeros(1, dtype=torch.int32))


def test_mechanisms_alone():
    from theroundtaible_amd.models.config import GroupedAttentionSpec, RotarySpec
    from theroundtaible_amd.ops import hybrid as Hy
    g = torch.Generator().manual_seed(3)
    T, W = 9, 20
    x = torch.randn(T, W, generator=g, dtype=torch.float64)
    w = 0.5 + torch.rand(W, generator=g, dtype=torch.float64)
    mu = torch.rand(W, generator=g, dtype=torch.float64)
    # norm + token shift, with a pending branch output, whole and cut in two with the state between
    y = torch.randn(T, W, generator=g, dtype=torch.float64)
    want = O.token_shift(O.rms_norm(x + y, w, 1e-5), mu)
    state = torch.zeros(1, W)
    got, xs = Hy.shift_norm(x.float(), y.float(), w.float(), 1e-5, mu.float(), state, *_one_span(T), torch.float32)
    torch.testing.assert_close(got.double(), want, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(xs.double(), x + y, rtol=1e-6, atol=1e-6)
    a, xa = Hy.shift_norm(x[:4].float(), None, w.float(), 1e-5, mu.float(), state, *_one_span(4), torch.float32)
    Hy.shift_state_update(xa, w.float(), 1e-5, state, torch.tensor([0, 4], dtype=torch.int32), torch.zeros(1, dtype=torch.int32))
    b, _ = Hy.shift_norm(x[4:].float(), None, w.float(), 1e-5, mu.float(), state, *_one_span(T - 4, 4), torch.float32)
    torch.testing.assert_close(torch.cat([a, b]).double(), O.token_shift(O.rms_norm(x, w, 1e-5), mu), rtol=1e-5, atol=1e-5)
    # frequencies and the rotation of pairs, on a part of the head only
    rot = {"base": 300.0, "dims": 6, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}}
    f = O.frequencies(rot)
    assert f[0] == 1.0 and f[2] < 300.0 ** (-4 / 6) * 0.99      # the slowest frequency is rescaled, the fastest kept
    table = Hy.rotary_table(RotarySpec(300.0, 6, ("llama3", 8.0, 1.0, 4.0, 64.0)), "cpu")
    torch.testing.assert_close(table.double(), f, rtol=1e-6, atol=0)
    v = torch.randn(7, 3, 10, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 50, 51, 1000, 4000])
    torch.testing.assert_close(Hy._rotate_pairs(v.float(), pos, table).double(), O.rotate_pairs(v, pos, f), rtol=1e-3, atol=1e-3)
    # queries / keys / values through the cache, then attention with sink and temperature
    H, G, D, E = 4, 2, 10, 6
    spec = GroupedAttentionSpec(H, G, D, E, 0.4, RotarySpec(300.0, 6, ("llama3", 8.0, 1.0, 4.0, 64.0)), sink=1.0, head_temp=True)
    proj = torch.randn(T, H * D + G * D + G * E, generator=g, dtype=torch.float64)
    temp = 0.5 + torch.rand(H, generator=g, dtype=torch.float64)
    kc, vc = torch.zeros(3, G, 4, D), torch.zeros(3, G, 4, E)
    bt = torch.tensor([[2, 0, 1]], dtype=torch.int32)
    slots = torch.tensor([bt[0, t // 4] * 4 + t % 4 for t in range(T)])
    q = Hy.qk_prep(proj.float(), spec, 0, H * D, (H + G) * D, table, 1e-5, torch.arange(T), kc, vc, slots, torch.float32)
    got = Hy.gqa_attention(q, kc, vc, bt, torch.tensor([0, T], dtype=torch.int32), torch.zeros(1, dtype=torch.int32), 0.4,
                           temp.float(), 1.0)
    qq = O.unit_rms(O.rotate_pairs(proj[:, :H * D].reshape(T, H, D), torch.arange(T), f), 1e-5)
    kk = O.unit_rms(O.rotate_pairs(proj[:, H * D:(H + G) * D].reshape(T, G, D), torch.arange(T), f), 1e-5)
    want = O.causal_attention(qq, kk, proj[:, (H + G) * D:].reshape(T, G, E), 0.4, temp, 1.0)
    torch.testing.assert_close(got.double().reshape(T, H, E), want, rtol=1e-4, atol=1e-5)
    # minGRU, whole and cut in two with the state between
    Wr = 13
    P = {"z": torch.randn(Wr, W, generator=g, dtype=torch.float64), "x": torch.randn(Wr, W, generator=g, dtype=torch.float64),
         "g": torch.randn(Wr, W, generator=g, dtype=torch.float64), "z.b": torch.randn(Wr, generator=g, dtype=torch.float64),
         "x.b": torch.randn(Wr, generator=g, dtype=torch.float64), "o": torch.eye(Wr, dtype=torch.float64)}
    want = O.min_gru(x, P, "")
    pr = torch.cat([x @ P["z"].T, x @ P["x"].T, x @ P["g"].T], 1).float()
    st = torch.zeros(1, Wr)
    cu = lambda n: torch.tensor([0, n], dtype=torch.int32)      # noqa: E731
    one = torch.zeros(1, dtype=torch.int32)
    a = Hy.mingru_scan(pr[:5], 0, Wr, 2 * Wr, Wr, P["z.b"].float(), P["x.b"].float(), st, cu(5), one * 0, one * 0, torch.float32)
    b = Hy.mingru_scan(pr[5:], 0, Wr, 2 * Wr, Wr, P["z.b"].float(), P["x.b"].float(), st, cu(T - 5), one * 0 + 5, one * 0, torch.float32)
    torch.testing.assert_close(torch.cat([a, b]).double(), want, rtol=1e-5, atol=1e-5)
    # clamped gated activation: values on both sides of every clamp
    gu = torch.tensor([[-3.0, 0.5, 2.0, 0.3, -3.0, 0.5, 2.0, -0.3]], dtype=torch.float64)
    Pf = {"gate": torch.eye(4, dtype=torch.float64), "up": torch.eye(4, dtype=torch.float64), "down": torch.eye(4, dtype=torch.float64)}
    want = O.feed_forward(gu[:, :4], dict(Pf, up=torch.diag(gu[0, 4:] / gu[0, :4])), "", 1.5)
    torch.testing.assert_close(Hy.limited_glu(gu.float(), 1.5, torch.float32).double(), want, rtol=1e-6, atol=1e-6)
    # the two-branch normed add
    xa, ya, yb = x.float().clone(), y.float(), torch.randn(T, W, generator=g)
    Hy.dual_norm_add_(xa, ya, w.float(), yb, mu.float(), 1e-5)
    torch.testing.assert_close(xa.double(), x + 0.5 * (O.rms_norm(y, w, 1e-5) + O.rms_norm(yb.double(), mu, 1e-5)), rtol=1e-5, atol=1e-5)


def test_config_reader_and_registry(tmp_path):
    cfg = make_config()
    make_checkpoint(tmp_path / "m", cfg)
    mc = get_config(str(tmp_path / "m"))
    assert mc.arch == "goganex" and mc.n_layers == 5 and mc.hidden == 40 and mc.embed_scale == 0.7
    assert [ls.source for ls in mc.layers] == [0, 1, 2, 1, 2] and [ls.ff for ls in mc.layers] == [56, 0, 56, 0, 56]
    a = mc.layers[1].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.rot.dims, a.sink, a.head_temp) == (4, 4, 10, 14, 6, 1.0, True)
    assert a.rot.scaling == ("llama3", 4.0, 1.0, 3.0, 48.0)
    p = mc.layers[2].mixer
    assert isinstance(p, ParallelSpec) and p.left.value_from_key and p.left.rot is None and p.right.width == 52
    assert mc.kv_bytes_per_token(2) == 2 * (2 * 24 + 2 * (4 * 24) + 2 * (3 * 16))
    assert mc.n_params() == sum(math.prod(s) for s, _, _ in layout_for(mc).values())
    for bad in (dict(cfg, loop={"start": 2, "stop": 5, "times": 2}),
                dict(cfg, layers=[dict(cfg["layers"][0], type="window")])):
        os.makedirs(tmp_path / "bad", exist_ok=True)
        json.dump(bad, open(tmp_path / "bad" / "config.json", "w"))
        with pytest.raises(ValueError):
            get_config(str(tmp_path / "bad"))
    tiny = get_config("tiny-goganex")
    assert [ls.source for ls in tiny.layers] == [0, 1, 2, 1, 2]


# ---- whole prompts, and the residual stream layer by layer ---------------------------------------

@pytest.mark.parametrize("run", RUNS)
def test_whole_prompt_and_layers(tmp_path, run):
    cfg = make_config()
    P = make_checkpoint(tmp_path / "m", cfg, seed=1)
    e = engine_for(tmp_path / "m", run)
    t = toks(45, cfg["vocab"], 1)
    want, layers = O.forward(t, P, cfg, return_layers=True)
    got = e.step([("a", t, list(range(len(t))))])
    close(got, want, run, "logits")
    # layer by layer through the model's own forward
    s = e.kv.seq("b")
    tok, pos, meta = e._varlen_meta([e.reserve(s, t)])
    keep = []
    with torch.no_grad():
        e.model.forward(tok, pos, e.kv, meta, keep_layers=keep)
    assert len(keep) == len(layers) == 5
    for i, (a, b) in enumerate(zip(keep, layers)):
        tol = 0.25 if run[1] == "bf16" else 1e-3
        assert float((a.double().cpu() - b).abs().max()) < tol, f"residual stream after layer run {i}"
    # residual adds fused into the next norm launch against separate adds
    e.model.fuse_adds = False
    close(e.step([("c", t, list(range(len(t))))]), want, run, "separate adds")


SHAPES = {
    # one query head per key/value head, and one key/value head for all query heads; no loop
    "groups": ([att(3, 3, 8), att(5, 1, 6, vdim=9), par(4, 1, 8, 17)], None),
    # heads wider than a wave's 64 lanes (keys and values), and a wide recurrence
    "wide": ([att(2, 1, 72, vdim=132, rot_dims=20, ff=0), par(2, 2, 80, 300)], None),
    # more query heads per key/value head than one attention workgroup's pairs
    "many-heads": ([att(40, 1, 4, ff=24)], None),
    # no frequency rescaling, rotation of a part of the head; a parallel layer first; layers
    # without feed-forward; a loop that covers everything three times
    "plain-rot": ([par(2, 1, 6, 8, ff=0), att(2, 2, 8, rot_dims=2, scaling=None, ff=0)], (0, 2, 3)),
    # a loop of one pass over one layer, constants that are 1
    "ones": ([att(1, 1, 4, ff=16, limit=1.0, scale=1.0), att(2, 1, 4)], (1, 2, 1)),
}


@pytest.mark.parametrize("run", RUNS)
@pytest.mark.parametrize("shape", list(SHAPES))
def test_other_sizes(tmp_path, run, shape):
    """Sizes and constants that the usual test model makes equal or 1."""
    layers, loop = SHAPES[shape]
    cfg = make_config(width=24, vocab=61, layers=layers, loop=loop, embed_scale=1.0 if shape == "ones" else 1.9)
    P = make_checkpoint(tmp_path / "m", cfg, seed=2)
    e = engine_for(tmp_path / "m", run, block_size=8)
    t = toks(70, cfg["vocab"], 2)
    want = O.forward(t, P, cfg)
    # a prompt portion, a portion of two tokens, then single tokens
    got = torch.cat([e.step([("a", t[:37], list(range(37)))]), e.step([("a", t[37:39], [0, 1])])] +
                    [e.step([("a", t[i:i + 1], [0])]) for i in range(39, 70)])
    close(got, want, run, shape)


# ---- portions, decoding, batches ------------------------------------------------------------------

@pytest.mark.parametrize("run", RUNS)
def test_prefill_against_token_by_token(tmp_path, run):
    cfg = make_config()
    P = make_checkpoint(tmp_path / "m", cfg, seed=3)
    e = engine_for(tmp_path / "m", run)
    t = toks(40, cfg["vocab"], 3)
    want = O.forward(t, P, cfg)
    one = torch.cat([e.step([("a", [x], [0])]) for x in t])          # from the first token on
    close(one, want, run, "token by token")
    whole = e.step([("b", t, list(range(40)))])
    close(whole, want, run, "whole")
    tol = 0.3 if run[1] == "bf16" else 1e-3
    assert float((one - whole).abs().max()) < tol


@pytest.mark.parametrize("run", RUNS)
@pytest.mark.parametrize("cuts", [[2, 2, 3, 1, 30, 2, 17, 1, 1, 5], [16, 16, 16, 16], [1, 63], [33, 31], [131, 2, 70]])
def test_portions(tmp_path, run, cuts):
    """Portions of several sizes, down to two tokens and one, cut inside and at page borders
    (pages of 16): the shift state and the recurrence state carry over every cut. The long portions
    take the recurrence's chunked scan on the GPU."""
    cfg = make_config()
    P = make_checkpoint(tmp_path / "m", cfg, seed=4)
    e = engine_for(tmp_path / "m", run)
    t = toks(sum(cuts), cfg["vocab"], 4)
    want = O.forward(t, P, cfg)
    out, at = [], 0
    for n in cuts:
        out.append(e.step([("a", t[at:at + n], list(range(n)))]))
        at += n
    close(torch.cat(out), want, run, f"portions {cuts}")


@pytest.mark.parametrize("run", RUNS)
def test_mixed_batch_equals_each_alone_and_slots_are_reused(tmp_path, run):
    """Unequal requests in one batch (portions beside single tokens, requests paused for a step),
    a pool of four state slots and few pages, so both are freed and used again."""
    cfg = make_config()
    P = make_checkpoint(tmp_path / "m", cfg, seed=5)
    e = engine_for(tmp_path / "m", run, tokens=160, slots=4)
    V = cfg["vocab"]
    reqs = {k: toks(n, V, 10 + i) for i, (k, n) in enumerate([("a", 50), ("b", 7), ("c", 33), ("d", 1), ("e", 41), ("f", 20)])}
    want = {k: O.forward(v, P, cfg) for k, v in reqs.items()}
    got = {k: [] for k in reqs}
    at = {k: 0 for k in reqs}
    plan = [[("a", 20), ("b", 7)], [("a", 1), ("c", 30), ("d", 1)], [("a", 2), ("c", 1)], [("c", 2), ("a", 27), ("e", 3)],
            [("e", 38), ("f", 5)], [("f", 1)], [("f", 14)]]
    for step in plan:
        entries, end = [], []
        for k, n in step:
            entries.append((k, reqs[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(reqs[k]):
                end.append(k)
        out = e.step(entries, end=end)
        o = 0
        for k, n in step:
            got[k].append(out[o:o + n])
            o += n
    for k in reqs:
        close(torch.cat(got[k]), want[k], run, f"request {k}")
    assert e.kv.alloc.num_free == e.kv.num_blocks and len(e.kv.state.free) == 4
    with pytest.raises(KVCacheOOM):       # a fifth live request has no slot
        for i in range(5):
            e.step([(f"x{i}", [1, 2], [])])


def _sharp_case(tmp_path, seed=8):
    """One attention layer with a sharp softmax (large score scale, temperatures above 1), 300
    tokens over many pages. Returns also, per head, the key the LAST query gives the most weight,
    that weight, and the share of the sink."""
    m = att(2, 1, 16, scale=4.0, ff=40)
    cfg = make_config(layers=[m], loop=None)

    def edit(P):
        P["l0.mix.temp"][:] = torch.tensor([1.5, 2.0])
    P = make_checkpoint(tmp_path / "m", cfg, seed=seed, edit=edit)
    t = toks(300, cfg["vocab"], seed)
    n = len(t)
    h = O.token_shift(O.rms_norm(P["embed"][torch.tensor(t)] * cfg["embedding"]["scale"], P["l0.norm1"], 1e-5), P["l0.shift"])
    f = O.frequencies(m["mixer"]["rot"])
    q = O.unit_rms(O.rotate_pairs((h @ P["l0.mix.q"].T).reshape(n, 2, 16), torch.arange(n), f), 1e-5)
    k = O.unit_rms(O.rotate_pairs((h @ P["l0.mix.k"].T).reshape(n, 1, 16), torch.arange(n), f), 1e-5)
    tops = []
    for hh in range(2):
        sc = (k[:, 0] @ q[-1, hh]) * 4.0 * float(P["l0.mix.temp"][hh])
        w = torch.softmax(torch.cat([sc, torch.zeros(1, dtype=torch.float64)]), 0)
        tops.append((int(w[:-1].argmax()), float(w[:-1].max()), float(w[-1])))
    return cfg, P, t, tops


@pytest.mark.parametrize("run", RUNS)
def test_far_key_and_sink_show(tmp_path, run):
    """The last query puts a large share of a head's softmax on ONE key far back, over several
    pages: a lost page, an off-by-one in the mask, a wrong temperature or a dropped sink changes
    these logits far beyond the tolerance. The sink's effect is shown by the oracle itself."""
    cfg, P, t, tops = _sharp_case(tmp_path)
    assert any(j < 250 and w > 0.2 for j, w, _ in tops), tops
    want = O.forward(t, P, cfg)
    e = engine_for(tmp_path / "m", run, tokens=1024)
    got = torch.cat([e.step([("a", t[:250], list(range(250)))])] + [e.step([("a", [x], [0])]) for x in t[250:]])
    close(got, want, run, "far key")


def test_sink_and_head_temperature_matter():
    """The oracle's attention with and without the sink, and with another temperature, differ by
    much more than any tolerance used here: the comparisons above would see either one missing."""
    g = torch.Generator().manual_seed(1)
    q, k, v = (torch.randn(12, 2, 8, generator=g, dtype=torch.float64) for _ in range(3))
    temp = torch.tensor([1.0, 2.0], dtype=torch.float64)
    a = O.causal_attention(q, k, v, 0.3, temp, 1.0)
    assert float((a - O.causal_attention(q, k, v, 0.3, temp, 0.0)).abs().max()) > 0.05
    assert float((a - O.causal_attention(q, k, v, 0.3, None, 1.0)).abs().max()) > 0.05
    # the first token sees itself and the sink: its weight is below one
    s = float((q[0, 0] @ k[0, 0]) * 0.3)
    torch.testing.assert_close(a[0, 0], v[0, 0] * math.exp(s) / (1 + math.exp(s)))


@pytest.mark.parametrize("run", RUNS)
@pytest.mark.parametrize("form", ["prompt", "decode"])
def test_one_key_stands_out_at_page_borders(run, form):
    """Attention alone on made-up queries and keys: one key's score is far above all others, so
    the output is that key's value. The key sits at the first position, on both sides of page
    borders, far back among hundreds, and at the query's own position; in a prompt's portion
    that starts inside a page and in single decoded rows with split keys."""
    from theroundtaible_amd.ops import hybrid as Hy
    dev, dt = run[0], torch.bfloat16 if run[1] == "bf16" else torch.float32
    H, G, D, E, BS, n = 4, 2, 16, 12, 8, 331
    g = torch.Generator().manual_seed(5)
    k = O.unit_rms(torch.randn(n, G, D, generator=g, dtype=torch.float64), 0.0)
    v = torch.randn(n, G, E, generator=g, dtype=torch.float64)
    nb = (n + BS - 1) // BS
    order = torch.randperm(nb, generator=g)          # pages in any order
    kc, vc = torch.zeros(nb, G, BS, D, dtype=dt), torch.zeros(nb, G, BS, E, dtype=dt)
    for t in range(n):
        kc[order[t // BS], :, t % BS] = k[t].to(dt)
        vc[order[t // BS], :, t % BS] = v[t].to(dt)
    targets = [0, 7, 8, 9, 63, 64, 200, 322, 323, n - 1]
    rows = list(range(n - len(targets), n)) if form == "prompt" else [n - 1] * len(targets)
    rows = [max(r, j) for r, j in zip(rows, targets)]
    q = torch.stack([torch.stack([k[j, h // 2] * 12.0 for h in range(H)]) for j in targets])      # [rows, H, D]
    kc, vc, bt = kc.to(dev), vc.to(dev), order.to(torch.int32)[None].to(dev)
    if form == "prompt":            # one span: consecutive rows n - len .. n - 1 (start inside a page)
        assert rows == list(range(n - len(targets), n))
        out = Hy.gqa_attention(q.to(dt).to(dev), kc, vc, bt, torch.tensor([0, len(rows)], dtype=torch.int32, device=dev),
                               torch.tensor([rows[0]], dtype=torch.int32, device=dev), 1.0, None, 1.0)
    else:                           # every row a sequence of its own over the same pages, keys split in 7 ranges
        B = len(rows)
        tiles = torch.stack([torch.arange(B), torch.arange(B)], 1).to(torch.int32).to(dev)
        out = Hy.gqa_attention(q.to(dt).to(dev), kc, vc, bt.expand(B, -1).contiguous(),
                               torch.arange(B + 1, dtype=torch.int32, device=dev),
                               torch.tensor(rows, dtype=torch.int32, device=dev), 1.0, None, 1.0, tiles=tiles,
                               num_splits=7 if dev != "cpu" else 1)
    out = out.double().cpu().reshape(len(rows), H, E)
    for i, (r, j) in enumerate(zip(rows, targets)):
        want = O.causal_attention(torch.cat([torch.zeros(r, H, D, dtype=torch.float64), q[i:i + 1]]), k[:r + 1], v[:r + 1],
                                  1.0, None, 1.0)[-1]
        tol = 0.05 if run[1] == "bf16" else 1e-4
        assert float((out[i] - want).abs().max()) < tol, f"row at {r}, key {j}"
        assert float((want - v[j].repeat_interleave(2, 0)).abs().max()) < 0.05     # the case shows that key


@pytest.mark.parametrize("run", RUNS)
def test_long_decoding_through_page_borders(tmp_path, run):
    cfg = make_config()
    P = make_checkpoint(tmp_path / "m", cfg, seed=7)
    e = engine_for(tmp_path / "m", run, block_size=8)
    t = toks(150, cfg["vocab"], 7)
    want = O.forward(t, P, cfg)
    got = torch.cat([e.step([("a", t[:5], list(range(5)))])] + [e.step([("a", [x], [0])]) for x in t[5:]])
    close(got, want, run, "long decode")


# ---- the engine's own generation path and scheduler -----------------------------------------------

def _greedy_oracle(P, cfg, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(O.forward(seq, P, cfg)[-1].argmax()))
    return seq[len(prompt):]


@pytest.mark.parametrize("run,graphs", [(("cpu", "fp32"), False), pytest.param(("cuda:0", "fp32"), False, marks=GPU),
                                        pytest.param(("cuda:0", "fp32"), True, marks=GPU)])
def test_greedy_generation_through_run_turns(tmp_path, run, graphs):
    """Greedy decoding through Engine.run_turns (tokenizer, prefix reuse, batched decode loop — the
    captured graph on the GPU) gives the oracle's tokens, for two requests of unequal length."""
    cfg = make_config(vocab=300, embed_scale=1.5)
    P = make_checkpoint(tmp_path / "m", cfg, seed=8)
    e = engine_for(tmp_path / "m", run, tokens=2048, graphs=graphs)
    sp = SamplingParams(temperature=0.0, max_new_tokens=12, ignore_eos=True, stop_on_consensus=False)
    prompts = ["De ridders aan de ronde tafel overleggen over het cachebeleid.", "Kort."]
    outs = e.run_turns([Turn("A", prompts[0], sp), Turn("B", prompts[1], sp)])
    for o, p in zip(outs, prompts):
        assert o.error is None, o.error
        ids = e.encode_prompt(p)
        assert o.ids == _greedy_oracle(P, cfg, ids, 12)
    # a second turn that extends the first one exactly reuses cache and state
    from theroundtaible_amd.prompt import Prompt
    p2 = Prompt().add(prompts[0]).add(outs[0].text, outs[0].ids, e.tokenizer.family)
    o2 = e.run_turns([Turn("A", p2, sp)])[0]
    ids2 = e.encode_prompt(prompts[0]) + outs[0].ids
    assert o2.ids == _greedy_oracle(P, cfg, ids2, 12)
    assert o2.metrics["reused_tokens"] in (0, len(ids2) - 1)


def test_rollback_restarts_a_stateful_sequence(tmp_path):
    """A prompt that diverges inside the resident sequence cannot keep the shift and recurrence
    states: the sequence restarts, and the result is still the oracle's."""
    cfg = make_config(vocab=300, embed_scale=1.5)
    P = make_checkpoint(tmp_path / "m", cfg, seed=9)
    e = engine_for(tmp_path / "m", ("cpu", "fp32"), tokens=2048)
    sp = SamplingParams(temperature=0.0, max_new_tokens=6, ignore_eos=True, stop_on_consensus=False)
    e.run_turns([Turn("A", "Een eerste lange vraag over de tafel.", sp)])
    o = e.run_turns([Turn("A", "Een eerste korte vraag.", sp)])[0]
    assert o.error is None and o.metrics["reused_tokens"] == 0
    assert o.ids == _greedy_oracle(P, cfg, e.encode_prompt("Een eerste korte vraag."), 6)


@GPU
def test_decode_steps_on_the_skinny_gemm(tmp_path):
    """Sizes the framework's skinny decode GEMM takes (K a multiple of 32, N of 16): decode steps
    run every linear of a layer on it, and the logits still match the oracle and the same steps on
    the library GEMM."""
    from theroundtaible_amd import ops
    if not ops.native_available():
        pytest.skip("main extension not built")
    cfg = make_config(width=64, vocab=80, layers=[att(4, 2, 16, ff=96), par(4, 2, 16, 64, ff=96)], loop=(0, 2, 2))
    P = make_checkpoint(tmp_path / "m", cfg, seed=11)
    t = toks(60, cfg["vocab"], 11)
    want = O.forward(t, P, cfg)
    outs = []
    for skinny in (True, False):
        e = engine_for(tmp_path / "m", ("cuda:0", "bf16"))
        e.model.use_skinny = skinny
        got = torch.cat([e.step([("a", t[:20], list(range(20)))])] + [e.step([("a", [x], [0])]) for x in t[20:]])
        close(got, want, ("cuda:0", "bf16"), f"skinny={skinny}")
        outs.append(got)
        if skinny:
            assert sorted(len(d) for d in e.model._dec.values()) == [4, 5]
    assert float((outs[0] - outs[1]).abs().max()) < 0.2


def test_serving_entry_points_match_run_turns():
    """The continuous-batching entry points (prefill + first token, then decode in chunks while the
    state follows) give the tokens of a single run_turns call; random-init preset weights."""
    def eng():
        return Engine(EngineConfig(model="tiny-goganex", weights="random:3", dtype="fp32", device="cpu",
                                   num_blocks=64, use_graphs=False, state_slots=4))
    sp = SamplingParams(temperature=0.0, max_new_tokens=10, ignore_eos=True, stop_on_consensus=False)
    turns = [Turn("A", "Eerste ridder spreekt over de cache.", sp), Turn("B", "Tweede.", sp)]
    want = [o.ids for o in eng().run_turns(turns)]
    e = eng()
    started = e.start_turns(turns)
    seqs = [s for s, _, _ in started]
    got = [[f] for _, f, _ in started]
    for steps in (4, 5):
        new = e.continue_decode(seqs, turns, [g[-1] for g in got], steps)
        for g, n in zip(got, new):
            g.extend(n)
    assert got == want
    assert all(s.state_len == s.length for s in seqs)


def test_grouped_cache_slots_rollback_and_fork():
    """The cache manager alone: per-layer shapes, slots handed out on first use and returned with
    the sequence; a roll-back keeps a stateful sequence only at its state's exact length; a fork
    copies both kinds of state."""
    from theroundtaible_amd.engine.kv_cache import GroupedKVCache
    kv = GroupedKVCache([(2, 6, 6), (1, 4, 10)], width=5, rec_widths=[0, 7], num_blocks=8, block_size=4, device="cpu",
                        dtype=torch.float32, n_slots=2)
    assert kv.k_layer(0).shape == (8, 2, 4, 6) and kv.v_layer(1).shape == (8, 1, 4, 10)
    assert kv.rec[0] is None and kv.rec[1].shape == (2, 7) and kv.shift[0].shape == (2, 5)
    assert GroupedKVCache.bytes_per_block(kv.shapes, 4, 4) == (24 + 14) * 4 * 4
    a = kv.seq("a")
    kv.ensure_capacity(a, 6)
    a.tokens.extend(range(6))
    assert kv.slot_of(a) == 0 and kv.slot_of(a) == 0
    a.state_len = 6
    kv.shift[1][a.slot].fill_(3.0)
    kv.rec[1][a.slot].fill_(2.0)
    b = kv.fork("a", "b")                       # shares pages, owns a copy of the state
    assert b.slot == 1 and b.state_len == 6 and float(kv.shift[1][b.slot].mean()) == 3.0 and float(kv.rec[1][b.slot].mean()) == 2.0
    with pytest.raises(KVCacheOOM):
        kv.slot_of(kv.seq("c"))                 # both slots are taken
    kv.truncate(a, 6)                           # the state's own length: kept
    assert a.length == 6
    kv.truncate(a, 4)                           # anything else: the sequence starts over
    assert a.length == 0 and a.state_len == 0 and a.blocks == []
    kv.free_seq("b")
    assert kv.slot_of(kv.seq("c")) == 1         # b's slot is used again
    kv.free_seq("a")
    kv.free_seq("c")
    assert kv.alloc.num_free == 8 and sorted(kv.state.free) == [0, 1]


@GPU
def test_layers_on_the_matrix_core_attention_kernels(tmp_path, monkeypatch):
    """Shapes the framework's bf16 matrix-core attention kernels take (pages of 32, heads of 64 and
    128, 1 to 4 query heads per key/value head): those layers keep their cache in the kernels'
    layout, pass the sink on and move the head temperature into the queries. Prompts in portions,
    a mixed batch and decode steps against the oracle and against the any-size kernel."""
    from theroundtaible_amd import ops
    from theroundtaible_amd.models.goganex import GoganexModel
    if not ops.native_available():
        pytest.skip("main extension not built")
    cfg = make_config(width=64, vocab=80, loop=(1, 3, 2),
                      layers=[att(4, 2, 64, ff=96, scale=0.2), par(2, 1, 128, 48, ff=0, scale=0.1),
                              att(3, 1, 128, ff=0, scale=0.15), att(4, 4, 24, ff=32)])
    P = make_checkpoint(tmp_path / "m", cfg, seed=12)
    ta, tb = toks(150, cfg["vocab"], 12), toks(70, cfg["vocab"], 13)
    wa, wb = O.forward(ta, P, cfg), O.forward(tb, P, cfg)
    run = ("cuda:0", "bf16")
    outs = []
    for matrix in (True, False):
        monkeypatch.setattr(GoganexModel, "matrix_attention", matrix)
        e = engine_for(tmp_path / "m", run, block_size=32, tokens=1024)
        assert e.kv.matrix == ([True, True, True, True, True, False] if matrix else [False] * 6)
        ga = [e.step([("a", ta[:100], list(range(100)))])]
        gb = []
        o = e.step([("a", ta[100:101], [0]), ("b", tb[:45], list(range(45)))])
        ga.append(o[:1]), gb.append(o[1:])
        o = e.step([("a", ta[101:131], list(range(30))), ("b", tb[45:46], [0])])
        ga.append(o[:30]), gb.append(o[30:])
        for i in range(19):
            o = e.step([("a", ta[131 + i:132 + i], [0]), ("b", tb[46 + i:47 + i], [0])])
            ga.append(o[:1]), gb.append(o[1:])
        gb.append(e.step([("b", tb[65:], list(range(5)))], end=["a", "b"]))
        ga, gb = torch.cat(ga), torch.cat(gb)
        close(ga, wa, run, f"a, matrix={matrix}")
        close(gb, wb, run, f"b, matrix={matrix}")
        outs.append((ga, gb))
    assert float((outs[0][0] - outs[1][0]).abs().max()) < 0.25
