"""Mupulorn through the engine (model registry, latent cache, state slots, Engine.step, generation)
against the plain float64 statement in ``oracle_mupulorn.py``, on small random checkpoints of
several shapes. Every case runs on the CPU (PyTorch statements of the ops) and, marked ``gpu``,
on the HIP kernels in fp32 and bf16.
"""
import json
import math
import os

import pytest
import torch
from safetensors.torch import save_file

import oracle_mupulorn as O
from theroundtaible_amd.engine import Engine, EngineConfig, SamplingParams, Turn
from theroundtaible_amd.engine.kv_cache import KVCacheOOM
from theroundtaible_amd.models.config import config_from_dir, get_config
from theroundtaible_amd.models.weights import layout_for

GPU = pytest.mark.gpu
RUNS = [("cpu", "fp32"), pytest.param(("cuda:0", "fp32"), marks=GPU), pytest.param(("cuda:0", "bf16"), marks=GPU)]


def mixer(heads, dim, rot_dim, vdim, kv_rank, q_rank, base=10000.0, rot_dims=None, scale=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
            "rot": {"base": base, "dims": rot_dim if rot_dims is None else rot_dims},
            "scale": (dim + rot_dim) ** -0.5 if scale is None else scale}


def make_config(width=48, vocab=97, taps=4, layers=None, logit_scale=0.5, softcap=20.0, eps=1e-5):
    if layers is None:
        a = {"type": "latent_attention", "mixer": mixer(3, 12, 6, 10, 24, 20), "mlp": {"kind": "dense", "ff": 56}}
        b = {"type": "latent_attention", "mixer": mixer(2, 8, 8, 16, 40, 12, base=500.0, rot_dims=4), "mlp": None}
        layers = [a, b, dict(a, weights_of=0)]
    return {"architecture": "Mupulorn", "canon": {"taps": taps}, "layers": layers, "logit_scale": logit_scale,
            "logit_softcap": softcap, "norm": {"eps": eps}, "vocab": vocab, "width": width}


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
        if name.endswith(("norm1", "norm2", "norm1b", "norm2b", "final.norm")):
            w = 0.6 + torch.rand(shape, generator=g)
        elif name.endswith(".norm"):
            w = 0.5 + torch.rand(shape, generator=g)
        elif name.endswith("mlp.act"):
            w = torch.tensor([0.8, -0.5, 0.3, 0.1])
        elif name.endswith(("canon1", "canon2")):
            w = torch.randn(shape, generator=g) * 0.4
        elif name.endswith("sink"):
            w = torch.randn(shape, generator=g)
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
        from theroundtaible_amd.ops import latent
        latent.native()     # the GPU cases fail loudly when the extension is missing
    return Engine(EngineConfig(model=str(path), weights=str(path), dtype=dtype, device=device, block_size=block_size,
                               num_blocks=(tokens + block_size - 1) // block_size + (1 if graphs else 0),
                               use_graphs=graphs, state_slots=slots, max_batch=slots))


def close(got, want, run, what=""):
    tol = dict(rtol=0, atol=0.35) if run[1] == "bf16" else dict(rtol=0, atol=2e-3)
    torch.testing.assert_close(got.double().cpu(), want, msg=lambda m: f"{what}: {m}", **tol)


def oracle_logits(P, cfg, tokens):
    return O.forward(tokens, P, cfg)


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


# ---- each mechanism alone (package ops on the CPU against the oracle's functions) ---------------

def test_mechanisms_alone():
    from theroundtaible_amd.ops import reference as ref
    g = torch.Generator().manual_seed(3)
    x = torch.randn(11, 20, generator=g, dtype=torch.float64)
    gain = torch.tensor(1.3, dtype=torch.float64)
    torch.testing.assert_close(ref.scalar_rms_norm(x.float(), gain.float(), 1e-5).double(), O.scalar_rms_norm(x, gain, 1e-5),
                               rtol=1e-5, atol=1e-6)
    for taps in (1, 2, 5):
        w = torch.randn(20, taps, generator=g, dtype=torch.float64)
        T = x.shape[0]
        meta = (torch.zeros(T, dtype=torch.int32), torch.arange(T), torch.zeros(1, dtype=torch.int32),
                torch.zeros(1, dtype=torch.int32))
        got = ref.canon_norm(x.float(), gain.float(), 1e-5, w.float(), torch.zeros(1, taps - 1, 20), *meta, torch.float32)
        torch.testing.assert_close(got.double(), O.input_conv(O.scalar_rms_norm(x, gain, 1e-5), w), rtol=1e-5, atol=1e-5)
    v = torch.randn(7, 3, 10, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 50, 51, 1000, 4000])
    torch.testing.assert_close(ref.rotate_interleaved(v.float(), pos, 300.0, 6).double(), O.rotate_pairs(v, pos, 300.0, 6),
                               rtol=1e-4, atol=1e-4)
    z = torch.randn(5, 33, generator=g, dtype=torch.float64)
    coef = torch.tensor([0.8, -0.5, 0.3, 0.1], dtype=torch.float64)
    torch.testing.assert_close(ref.poly_norm(z.float(), coef.float(), 1e-5, torch.float32).double(), O.poly_norm(z, coef, 1e-5),
                               rtol=1e-5, atol=1e-5)


def test_config_reader_and_registry(tmp_path):
    cfg = make_config()
    make_checkpoint(tmp_path / "m", cfg)
    mc = get_config(str(tmp_path / "m"))
    assert mc.arch == "mupulorn" and mc.n_layers == 3 and mc.canon_taps == 4 and mc.hidden == 48
    assert [ls.source for ls in mc.layers] == [0, 1, 0] and [ls.ff for ls in mc.layers] == [56, 0, 56]
    assert mc.layers[1].mixer.rot_dims == 4 and mc.layers[1].mixer.rot_base == 500.0
    assert mc.kv_bytes_per_token(2) == 2 * (30 + 48 + 30)
    bad = dict(cfg, architecture="Nope")
    os.makedirs(tmp_path / "bad")
    json.dump(bad, open(tmp_path / "bad" / "config.json", "w"))
    with pytest.raises(KeyError):
        get_config(str(tmp_path / "bad"))
    assert get_config("tiny-mupulorn").layers[1].source == 0


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
    for i, (a, b) in enumerate(zip(keep, layers)):
        tol = 0.25 if run[1] == "bf16" else 1e-3
        assert float((a.double().cpu() - b).abs().max()) < tol, f"residual stream after layer {i}"


@pytest.mark.parametrize("run", RUNS)
@pytest.mark.parametrize("shape", ["one-head", "wide", "taps1", "no-rot-tail", "tiles"])
def test_other_sizes(tmp_path, run, shape):
    """Sizes that the usual test model makes equal or 1: a single head, rows wider than a key
    tile's lanes, one tap (no state), rotation on a part of the rotary entries only."""
    lay = {"one-head": [{"type": "latent_attention", "mixer": mixer(1, 16, 4, 8, 16, 8), "mlp": {"kind": "dense", "ff": 24}}],
           "wide": [{"type": "latent_attention", "mixer": mixer(5, 24, 10, 12, 136, 36), "mlp": None},
                    {"type": "latent_attention", "mixer": mixer(9, 8, 2, 8, 72, 16), "mlp": {"kind": "dense", "ff": 200}}],
           # latents of 64 and 128 with rotary parts of 16 and 32 (the shapes the bf16 matrix-core
           # attention takes) beside one it does not take, and a layer that shares the first one's weights
           "tiles": [{"type": "latent_attention", "mixer": mixer(4, 32, 16, 24, 64, 48), "mlp": {"kind": "dense", "ff": 72}},
                     {"type": "latent_attention", "mixer": mixer(6, 16, 32, 16, 128, 40, base=300.0), "mlp": None},
                     {"type": "latent_attention", "mixer": mixer(3, 16, 8, 16, 96, 24), "mlp": {"kind": "dense", "ff": 40}},
                     {"type": "latent_attention", "mixer": mixer(4, 32, 16, 24, 64, 48), "mlp": {"kind": "dense", "ff": 72},
                      "weights_of": 0}],
           "taps1": None, "no-rot-tail": [{"type": "latent_attention", "mixer": mixer(2, 6, 7, 5, 18, 10, rot_dims=2),
                                           "mlp": {"kind": "dense", "ff": 30}}]}[shape]
    cfg = make_config(width=40, vocab=61, taps=1 if shape == "taps1" else 3, layers=lay, logit_scale=1.0, softcap=8.0)
    P = make_checkpoint(tmp_path / "m", cfg, seed=2)
    e = engine_for(tmp_path / "m", run, block_size=8)
    t = toks(70, cfg["vocab"], 2)
    want = oracle_logits(P, cfg, t)
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
    want = oracle_logits(P, cfg, t)
    one = torch.cat([e.step([("a", [x], [0])]) for x in t])          # from the first token on
    close(one, want, run, "token by token")
    whole = e.step([("b", t, list(range(40)))])
    close(whole, want, run, "whole")
    tol = 0.3 if run[1] == "bf16" else 1e-3
    assert float((one - whole).abs().max()) < tol


@pytest.mark.parametrize("run", RUNS)
@pytest.mark.parametrize("cuts", [[2, 2, 3, 1, 30, 2, 17, 1, 1, 5], [16, 16, 16, 16], [1, 63], [33, 31]])
def test_portions(tmp_path, run, cuts):
    """Portions of several sizes, down to two tokens and one, cut inside and at page borders
    (pages of 16) and shorter than the convolution's reach."""
    cfg = make_config()
    P = make_checkpoint(tmp_path / "m", cfg, seed=4)
    e = engine_for(tmp_path / "m", run)
    t = toks(sum(cuts), cfg["vocab"], 4)
    want = oracle_logits(P, cfg, t)
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
    want = {k: oracle_logits(P, cfg, v) for k, v in reqs.items()}
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


def _far_key_case(tmp_path, seed=8):
    """One layer with a sharp softmax (large score scale) and strong sinks, 300 tokens over many
    pages. Returns also, per head, the key the LAST query gives the most weight and that weight."""
    m = mixer(2, 16, 8, 12, 24, 16, scale=1.2)
    cfg = make_config(layers=[{"type": "latent_attention", "mixer": m, "mlp": {"kind": "dense", "ff": 40}}])

    def edit(P):
        P["l0.mix.sink"][:] = torch.tensor([24.0, 20.0])
    P = make_checkpoint(tmp_path / "m", cfg, seed=seed, edit=edit)
    t = toks(300, cfg["vocab"], seed)
    h = O.input_conv(O.scalar_rms_norm(P["embed"][torch.tensor(t)], P["l0.norm1"], 1e-5), P["l0.canon1"])
    qs, ks, _ = O.latent_qkv(h, P, "l0.mix.", m, 1e-5)
    tops = []
    for hh in range(2):
        sc = (ks[hh] @ qs[hh, -1]) * m["scale"]
        w = torch.softmax(torch.cat([sc, P["l0.mix.sink"][hh:hh + 1]]), 0)
        tops.append((int(w[:-1].argmax()), float(w[:-1].max()), float(w[-1])))
    return cfg, P, t, tops


@pytest.mark.parametrize("run", RUNS)
def test_far_key_and_sink_show(tmp_path, run):
    """The last query puts most of a head's softmax on ONE key more than a hundred positions and
    several pages back, and the sinks hold a visible share: a lost page, an off-by-one in the
    mask or a dropped sink changes these logits far beyond the tolerance."""
    cfg, P, t, tops = _far_key_case(tmp_path)
    # the case shows a far key and, on the same head, the sink
    assert any(j < 190 and w > 0.3 and 0.02 < sk < 0.9 for j, w, sk in tops), tops
    want = oracle_logits(P, cfg, t)
    e = engine_for(tmp_path / "m", run, tokens=1024)
    got = torch.cat([e.step([("a", t[:250], list(range(250)))])] + [e.step([("a", [x], [0])]) for x in t[250:]])
    close(got, want, run, "far key")


@pytest.mark.parametrize("run", RUNS)
def test_long_decoding_through_page_borders(tmp_path, run):
    cfg = make_config(taps=3)
    P = make_checkpoint(tmp_path / "m", cfg, seed=7)
    e = engine_for(tmp_path / "m", run, block_size=8)
    t = toks(150, cfg["vocab"], 7)
    want = oracle_logits(P, cfg, t)
    got = torch.cat([e.step([("a", t[:5], list(range(5)))])] + [e.step([("a", [x], [0])]) for x in t[5:]])
    close(got, want, run, "long decode")


# ---- the engine's own generation path and scheduler -----------------------------------------------

def _greedy_oracle(P, cfg, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(oracle_logits(P, cfg, seq)[-1].argmax()))
    return seq[len(prompt):]


@pytest.mark.parametrize("run,graphs", [(("cpu", "fp32"), False), pytest.param(("cuda:0", "fp32"), False, marks=GPU),
                                        pytest.param(("cuda:0", "fp32"), True, marks=GPU)])
def test_greedy_generation_through_run_turns(tmp_path, run, graphs):
    """Greedy decoding through Engine.run_turns (tokenizer, prefix reuse, batched decode loop — the
    captured graph on the GPU) gives the oracle's tokens, for two requests of unequal length."""
    cfg = make_config(vocab=300, logit_scale=2.0, softcap=50.0)
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
    """A prompt that diverges inside the resident sequence cannot keep the convolution state: the
    sequence restarts, and the result is still the oracle's."""
    cfg = make_config(vocab=300, logit_scale=2.0, softcap=50.0)
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
    run all five linears of a layer on it, and the logits still match the oracle and the same
    steps on the library GEMM."""
    from theroundtaible_amd import ops
    if not ops.native_available():
        pytest.skip("main extension not built")
    lay = [{"type": "latent_attention", "mixer": mixer(2, 16, 16, 16, 64, 32), "mlp": {"kind": "dense", "ff": 96}}] * 2
    cfg = make_config(width=64, vocab=80, layers=lay)
    P = make_checkpoint(tmp_path / "m", cfg, seed=11)
    t = toks(60, cfg["vocab"], 11)
    want = oracle_logits(P, cfg, t)
    outs = []
    for skinny in (True, False):
        e = engine_for(tmp_path / "m", ("cuda:0", "bf16"))
        e.model.use_skinny = skinny
        got = torch.cat([e.step([("a", t[:20], list(range(20)))])] + [e.step([("a", [x], [0])]) for x in t[20:]])
        close(got, want, ("cuda:0", "bf16"), f"skinny={skinny}")
        outs.append(got)
        if skinny:
            assert all(len(d) == 5 for d in e.model._dec.values())
    assert float((outs[0] - outs[1]).abs().max()) < 0.2


def test_serving_entry_points_match_run_turns():
    """The continuous-batching entry points (prefill + first token, then decode in chunks while the
    state follows) give the tokens of a single run_turns call; random-init preset weights."""
    def eng():
        return Engine(EngineConfig(model="tiny-mupulorn", weights="random:3", dtype="fp32", device="cpu",
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


def test_latent_cache_slots_rollback_and_fork():
    """The cache manager alone: slots are handed out on first use and come back with the sequence;
    a roll-back keeps a stateful sequence only at its state's exact length; a fork copies the state."""
    from theroundtaible_amd.engine.kv_cache import LatentKVCache
    kv = LatentKVCache([10, 6], conv_width=4, taps=3, num_blocks=8, block_size=4, device="cpu",
                       dtype=torch.float32, n_slots=2)
    a = kv.seq("a")
    kv.ensure_capacity(a, 6)
    a.tokens.extend(range(6))
    assert kv.slot_of(a) == 0 and kv.slot_of(a) == 0
    a.state_len = 6
    kv.conv[1][a.slot].fill_(3.0)
    b = kv.fork("a", "b")                       # shares pages, owns a copy of the state
    assert b.slot == 1 and b.state_len == 6 and float(kv.conv[1][b.slot].mean()) == 3.0
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
    assert kv.layer_rows(0).shape == (8, 4, 10) and kv.layer_rows(1).shape == (8, 4, 6)
