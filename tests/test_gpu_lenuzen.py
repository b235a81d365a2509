"""MI355X: the layer-list engine serving Lenuzen models against the plain float64 restatement
in tests/lenuzen_ref.py, on small random models made here.

Errors are per position: || got - ref || / || ref || over the vocabulary. With f32 matrices
the engine differs from the restatement by f32 rounding only (F32_TOL); with bf16 matrices by
the rounding of the products' inputs and of the cached keys and values (BF16_TOL). A lost key,
a window one token off, a missing sink or a token one place off moves the logits by orders of
magnitude more than F32_TOL; the edge tests show that on their own models before they trust it.
"""
import copy
import json
import os
import subprocess

import numpy as np
import pytest

import lenuzen_cases as C
import lenuzen_ref as R

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F32_TOL, BF16_TOL = 2e-4, 6e-2


@pytest.fixture(scope="module")
def rt():
    from yalm_amd import runtime

    runtime.check(runtime.lib.yalm_set_device(0))
    return runtime


def build(rt, cfg, wdt, seed=0, max_tokens=512, tensors=None):
    from yalm_amd import layered as Ly

    t = tensors if tensors is not None else Ly.lenuzen_random_tensors(cfg, seed=seed)
    c = Ly.lenuzen_config(cfg, max_tokens=max_tokens, weight_dtype=wdt)
    model = rt.SeqModel.from_packed(c, Ly.lenuzen_pack(c, t))
    return model, rt.SeqDecoder(model), {k: v.astype(np.float64) for k, v in t.items()}


def rel_err(got, ref):
    return np.linalg.norm(got - ref, axis=-1) / np.linalg.norm(ref, axis=-1)


def tol(dtype):
    return F32_TOL if dtype == "f32" else BF16_TOL


def wdt_of(dtype):
    from yalm_amd import models as M

    return M.F32 if dtype == "f32" else M.BF16


def run_portions(dec, tok, sizes):
    """Feed tok in portions of the given sizes (the last one takes the rest), asking for
    every position's logits."""
    out, at = [], 0
    for s in list(sizes) + [len(tok)]:
        s = min(s, len(tok) - at)
        if s <= 0:
            break
        out.append(dec.step(tok[at:at + s], list(range(s))))
        at += s
    return np.concatenate(out)


ALONE = {"window": C.ONLY_WINDOW, "chunk": C.ONLY_CHUNK, "dense": C.ONLY_DENSE}


@pytest.mark.parametrize("name", sorted(ALONE))
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_each_mechanism_alone(rt, name, dtype):
    cfg = ALONE[name]
    model, dec, w = build(rt, cfg, wdt_of(dtype), seed=1)
    try:
        tok = C.tokens(cfg, 70, 1)
        ref = R.forward(cfg, w, tok)
        assert rel_err(dec.step(tok, list(range(len(tok)))), ref).max() < tol(dtype)
        dec.reset()
        assert rel_err(run_portions(dec, tok, [30] + [1] * 40), ref).max() < tol(dtype)
    finally:
        dec.close()
        model.close()


@pytest.mark.parametrize("cfg", [C.MIXED, C.ODD, C.WIDE, C.TILED], ids=["mixed", "odd", "wide", "tiled"])
def test_residual_stream_after_every_layer(rt, cfg):
    from yalm_amd import models as M

    model, dec, w = build(rt, cfg, M.F32, seed=2)
    try:
        tok = C.tokens(cfg, 57, 2)
        layers = []
        R.forward(cfg, w, tok, layers_out=layers)
        dec.layer_dump(True)
        dec.step(tok)
        got = dec.get_layers(len(tok))
        for i, ref in enumerate(layers):
            e = np.abs(got[i] - ref).max() / np.abs(ref).max()
            assert e < 1e-4, f"layer {i}: {e}"
    finally:
        dec.close()
        model.close()


@pytest.mark.parametrize("cfg", [C.MIXED, C.ODD, C.WIDE, C.TILED], ids=["mixed", "odd", "wide", "tiled"])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_prefill_then_token_by_token(rt, cfg, dtype):
    """A prompt in one step, then single tokens through the caches: windows and chunks pass
    over decoded tokens, long prompts take the portion kernels."""
    model, dec, w = build(rt, cfg, wdt_of(dtype), seed=3, max_tokens=700)
    try:
        n = 420 if cfg in (C.WIDE, C.TILED) else 150
        tok = C.tokens(cfg, n, 3)
        ref = R.forward(cfg, w, tok)
        got = run_portions(dec, tok, [n - 60] + [1] * 60)
        assert rel_err(got, ref).max() < tol(dtype)
        dec.reset()
        assert rel_err(dec.step(tok, list(range(n))), ref).max() < tol(dtype)
    finally:
        dec.close()
        model.close()


PORTIONS = [[2] * 30, [3, 2, 9, 8, 2, 64, 65], [1, 2, 3, 4, 5, 6, 7, 8, 9, 10], [128, 2, 2, 1, 40], [7, 200]]


@pytest.mark.parametrize("cfg", [C.MIXED, C.ODD, C.WIDE], ids=["mixed", "odd", "wide"])
@pytest.mark.parametrize("sizes", PORTIONS, ids=[str(i) for i in range(len(PORTIONS))])
def test_portions_of_any_size(rt, cfg, sizes):
    """Portions cut anywhere (inside windows and chunks, down to two tokens) against the
    whole sequence; the GEMV / tile switch (8 | 9 tokens) and tile edges (64 | 65) included."""
    from yalm_amd import models as M

    model, dec, w = build(rt, cfg, M.F32, seed=4)
    try:
        tok = C.tokens(cfg, 260, 4)
        ref = R.forward(cfg, w, tok)
        assert rel_err(run_portions(dec, tok, sizes), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_portions_bf16_differ_by_rounding_only(rt):
    from yalm_amd import models as M

    cfg = C.TILED
    model, dec, w = build(rt, cfg, M.BF16, seed=5, max_tokens=700)
    try:
        tok = C.tokens(cfg, 600, 5)
        ref = R.forward(cfg, w, tok)
        for sizes in ([600], [300, 2, 170, 1, 1, 1], [64] * 9):
            dec.reset()
            assert rel_err(run_portions(dec, tok, sizes), ref).max() < BF16_TOL
    finally:
        dec.close()
        model.close()


def test_decoder_reused_after_reset(rt):
    """Cache rows of an ended sequence must not leak into the next one: the second sequence
    on a reused decoder equals the same sequence on a fresh decoder bit for bit."""
    from yalm_amd import models as M

    cfg = C.MIXED
    model, dec, w = build(rt, cfg, M.F32, seed=8)
    fresh = rt.SeqDecoder(model)
    try:
        a, b = C.tokens(cfg, 90, 6), C.tokens(cfg, 41, 7)
        run_portions(dec, a, [50, 1, 1, 38])
        dec.reset()
        assert dec.pos == 0
        got = run_portions(dec, b, [20, 1, 20])
        want = run_portions(fresh, b, [20, 1, 20])
        assert np.array_equal(got, want)
        assert rel_err(got, R.forward(cfg, w, b)).max() < F32_TOL
    finally:
        dec.close()
        fresh.close()
        model.close()


def test_two_live_sequences_do_not_mix(rt):
    """Two decoders on one model, unequal requests, their steps interleaved: each equals its
    sequence alone."""
    from yalm_amd import models as M

    cfg = C.MIXED
    model, d1, w = build(rt, cfg, M.F32, seed=20)
    d2 = rt.SeqDecoder(model)
    try:
        a, b = C.tokens(cfg, 60, 20), C.tokens(cfg, 45, 21)
        ga, gb, ia, ib = [], [], 0, 0
        for sa, sb in ((20, 3), (1, 30), (9, 1), (30, 11)):
            ga.append(d1.step(a[ia:ia + sa], list(range(sa))))
            gb.append(d2.step(b[ib:ib + sb], list(range(sb))))
            ia, ib = ia + sa, ib + sb
        assert rel_err(np.concatenate(ga), R.forward(cfg, w, a)).max() < F32_TOL
        assert rel_err(np.concatenate(gb), R.forward(cfg, w, b)).max() < F32_TOL
    finally:
        d1.close()
        d2.close()
        model.close()


def _resized(cfg, delta):
    c = copy.deepcopy(cfg)
    c["layers"][0]["mixer"]["mask"]["size"] += delta
    return c


EDGE = {
    # peaked attention (large score scale) in one layer: single keys decide positions
    "window": C.config([("attention", C.window(heads=2, kv_heads=1, dim=16, vdim=24, size=37, scale=2.5, rot_dims=8), None)],
                       width=64, vocab=101),
    "chunk": C.config([("attention_2", C.chunk(heads=2, kv_heads=2, dim=16, vdim=24, size=29, scale=2.5, rot_dims=16), None)],
                      width=64, vocab=101),
    # a window longer than several key tiles: winning keys hundreds of positions back
    "far": C.config([("attention", C.window(heads=2, kv_heads=1, dim=16, vdim=24, size=333, scale=2.5, rot_dims=8), None)],
                    width=64, vocab=101),
}


@pytest.mark.parametrize("name", ["window", "chunk"])
def test_keys_just_inside_and_just_outside_an_edge(rt, name):
    """The restatement with the mask one position shorter / longer names the positions where
    the key just inside / just outside the edge decides the logits (they differ there by far
    more than the tolerance); the engine must agree with the true size at all of them, with
    the query in a prompt's portion and decoded alone."""
    from yalm_amd import models as M

    cfg = EDGE[name]
    model, dec, w = build(rt, cfg, M.F32, seed=9)
    try:
        tok = C.tokens(cfg, 240, 8)
        ref = R.forward(cfg, w, tok)
        inside = rel_err(R.forward(_resized(cfg, -1), w, tok), ref)   # the edge key taken away
        outside = rel_err(R.forward(_resized(cfg, +1), w, tok), ref)  # the next key let in
        assert (inside > 100 * F32_TOL).sum() >= 5 and (outside > 100 * F32_TOL).sum() >= 5
        for sizes in ([240], [100] + [1] * 140, [61, 2, 50, 2, 2, 93]):
            dec.reset()
            assert rel_err(run_portions(dec, tok, sizes), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_far_keys_decide_the_output(rt):
    """The restatement's own softmax weights name late queries whose winning key lies more
    than 250 positions back, inside the window; changing THAT token must move the query's
    logits, and the engine must follow, in a prompt's portion and decoded alone."""
    from yalm_amd import models as M

    cfg = EDGE["far"]
    model, dec, w = build(rt, cfg, M.F32, seed=10, max_tokens=600)
    try:
        a = C.tokens(cfg, 500, 9)
        P = []
        ra = R.forward(cfg, w, a, weights_out=P)
        P = P[0]
        far = [(P[h, t].max(), t, int(P[h, t].argmax())) for h in range(2) for t in range(340, 500)
               if t - int(P[h, t].argmax()) >= 250]
        assert far, "no late query with a far winning key: pick another seed"
        weight, t, j = max(far)
        assert weight > 0.5
        b = list(a)
        b[j] = (b[j] + 17) % cfg["vocab"]
        rb = R.forward(cfg, w, b)
        assert rel_err(ra[t], rb[t]) > 100 * F32_TOL
        for tok, ref in ((a, ra), (b, rb)):
            for sizes in ([490], [t] + [1] * 5):
                dec.reset()
                assert rel_err(run_portions(dec, tok, sizes), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_sink_and_score_mixing_show_in_the_logits(rt):
    """Without the sink's 1 in the denominator, or with the identity in place of the mixing
    matrix, the restatement moves far beyond the tolerance: the engine agreeing with the
    restatement means it computes both."""
    from yalm_amd import models as M

    cfg = C.ONLY_CHUNK
    model, dec, w = build(rt, cfg, M.F32, seed=11)
    try:
        tok = C.tokens(cfg, 40, 10)
        ref = R.forward(cfg, w, tok)
        w2 = dict(w)
        w2["l0.mix.talk"] = np.eye(w["l0.mix.talk"].shape[0])
        assert rel_err(R.forward(cfg, w2, tok), ref).max() > 100 * F32_TOL
        keep = R.softmax_rows
        try:
            R.softmax_rows = lambda s, mask, sink: keep(s, mask, False)
            assert rel_err(R.forward(cfg, w, tok), ref).max() > 100 * F32_TOL
        finally:
            R.softmax_rows = keep
        assert rel_err(dec.step(tok, list(range(40))), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


@pytest.mark.parametrize("n", [1, 2, 3, 5])
def test_first_tokens(rt, n):
    from yalm_amd import models as M

    cfg = C.MIXED
    model, dec, w = build(rt, cfg, M.F32, seed=12)
    try:
        tok = C.tokens(cfg, n, 9)
        ref = R.forward(cfg, w, tok)
        assert rel_err(dec.step(tok, list(range(n))), ref).max() < F32_TOL
        dec.reset()
        assert rel_err(run_portions(dec, tok, [1] * n), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


@pytest.mark.parametrize("cfg", [C.ODD, C.MIXED], ids=["odd", "mixed"])
def test_long_decoding(rt, cfg):
    """200 single tokens: every window and chunk of the model passes over decoded tokens
    several times."""
    from yalm_amd import models as M

    model, dec, w = build(rt, cfg, M.F32, seed=13)
    try:
        tok = C.tokens(cfg, 5 + 200, 10)
        got = run_portions(dec, tok, [5] + [1] * 200)
        assert rel_err(got, R.forward(cfg, w, tok)).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_greedy_generation(rt):
    """The device greedy loop (no host round trip) picks the restatement's tokens, and the
    sequence can be continued by ordinary steps afterwards."""
    from yalm_amd import models as M

    cfg = C.MIXED
    model, dec, w = build(rt, cfg, M.F32, seed=14)
    try:
        prompt = C.tokens(cfg, 12, 11)
        dec.step(prompt[:-1])
        gen = dec.generate_greedy(prompt[-1], 40)
        seq = list(prompt)
        for g in gen:
            lg = R.forward(cfg, w, seq)[-1]
            top2 = np.sort(lg)[-2:]
            assert top2[1] - top2[0] > 1e-3, "the test's model has a near tie; pick another seed"
            assert int(np.argmax(lg)) == g
            seq.append(g)
        assert dec.pos == len(prompt) - 1 + len(gen)
        nxt = dec.step([gen[-1]], [0])
        assert rel_err(nxt, R.forward(cfg, w, seq)[-1:]).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_greedy_graph_replays_match_eager_steps(rt):
    """The greedy loop replays one captured token graph. Several generate calls with ordinary
    (eager) steps and synchronisations between them: every replayed token equals the argmax of
    an eager step of a second decoder fed the same tokens."""
    from yalm_amd import models as M

    cfg = C.MIXED
    model, dec, w = build(rt, cfg, M.BF16, seed=15)
    eager = rt.SeqDecoder(model)
    try:
        prompt = C.tokens(cfg, 9, 16)
        dec.step(prompt[:-1])
        eager.step(prompt[:-1])
        tok = prompt[-1]
        for n in (3, 1, 6, 2):
            gen = dec.generate_greedy(tok, n)
            for g in gen:
                lg = eager.step([tok], [0])[0]
                assert int(np.argmax(lg)) == g
                tok = g
            extra = C.tokens(cfg, 2, 17 + n)
            a = dec.step(extra, [1])
            b = eager.step(extra, [1])
            assert np.array_equal(a, b)
            tok = int(np.argmax(a[0]))
        assert dec.pos == eager.pos
    finally:
        dec.close()
        eager.close()
        model.close()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_attention_options_combine_freely(rt, dtype):
    """The attention mixer's options are parameters of the engine, not of one design: a layer
    put together by hand (full causal mask, no query / key norm, unit-rms values, a sink, head
    temperatures, rotation over the whole head without rescaling, no gate, no mixing) inside
    the other envelope (rms norms, an opening norm per sublayer, an untied head) against the
    same combination restated from the per-mechanism functions."""
    from yalm_amd import layered as Ly

    W, V_, H, G, D, Vd, T = 48, 67, 4, 2, 16, 24, 90
    rng = np.random.default_rng(5)

    def rnd(*shape, s=None):
        a = rng.standard_normal(shape) * (s if s is not None else 1.0 / np.sqrt(shape[-1]))
        return Ly.bf16_to_f32(Ly.f32_to_bf16(a.astype(np.float32))).reshape(shape)

    t = {"embed": rnd(V_, W, s=0.1), "head": rnd(V_, W), "q": rnd(H * D, W), "k": rnd(G * D, W), "v": rnd(G * Vd, W),
         "o": rnd(W, H * Vd), "norm1": 1 + rnd(W, s=0.2), "norm1b": 1 + rnd(W, s=0.2), "final": 1 + rnd(W, s=0.2),
         "temp": np.float32(1.0) + np.abs(rnd(H, s=0.5))}
    spec = Ly.LayerSpec(Ly.MIX_ATTN, heads=H, kv_heads=G, dim=D, vdim=Vd, attn_scale=0.8, mask_kind=Ly.MASK_CAUSAL,
                        qk_norm=Ly.QK_NONE, v_norm=1, sink=1, rot_dims=D, rot_base=100.0, head_temps=True)
    c = Ly.LayeredConfig("by hand", W, V_, [spec], embed_scale=3.0, norm_eps=1e-5, max_tokens=128, weight_dtype=wdt_of(dtype),
                         norm_kind=Ly.NORM_RMS, pre_norm=True, pos_embed=False, logit_scale=1.25)
    as_w = (lambda a: np.ascontiguousarray(a, np.float32)) if dtype == "f32" else Ly.f32_to_bf16
    layer = {"norm1": t["norm1"], "norm1b": t["norm1b"], "w_in": as_w(np.concatenate([t["q"], t["k"], t["v"]])),
             "w_o": as_w(t["o"]), "head_temp": t["temp"]}
    assert set(layer) == set(Ly.packed_shapes(c, spec))
    model = rt.SeqModel.from_packed(c, {"embed": as_w(t["embed"]), "final_norm": t["final"], "head": as_w(t["head"]),
                                        "layers": [layer]})
    dec = rt.SeqDecoder(model)
    try:
        w = {k: v.astype(np.float64) for k, v in t.items()}
        tok = rng.integers(0, V_, T).tolist()
        eps = 1e-5
        x = w["embed"][tok] * 3.0
        h = R.unit_rms(x, eps) * w["norm1"]
        rot = {"dims": D, "base": 100.0}
        pos = np.arange(T)
        q = R.rotate((h @ w["q"].T).reshape(T, H, D), rot, pos)
        k = R.rotate((h @ w["k"].T).reshape(T, G, D), rot, pos)
        v = R.unit_rms((h @ w["v"].T).reshape(T, G, Vd), eps)
        o, _ = R.attention_core(q, k, v, 0.8, R.visible("causal", 0, T), temp=w["temp"], sink=True)
        x = x + R.unit_rms(o.reshape(T, H * Vd) @ w["o"].T, eps) * w["norm1b"]
        ref = (R.unit_rms(x, eps) * w["final"]) @ w["head"].T * 1.25
        assert rel_err(dec.step(tok, list(range(T))), ref).max() < tol(dtype)
        dec.reset()
        assert rel_err(run_portions(dec, tok, [40, 2, 9] + [1] * 39), ref).max() < tol(dtype)
    finally:
        dec.close()
        model.close()


_LONG_REF = {}


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_prompt_longer_than_one_internal_portion(rt, dtype):
    """A step of more tokens than the engine's work buffers hold (4096) is cut inside the
    engine, in the middle of a window and of a chunk; asked rows on both sides of the cut
    come back in order."""
    cfg = C.config([("attention", C.window(heads=2, kv_heads=1, dim=8, vdim=8, size=150, rot_dims=4, scale=0.35), None),
                    ("attention_2", C.chunk(heads=2, kv_heads=2, dim=8, vdim=8, size=1000, rot_dims=8, scale=0.35), None)],
                   width=32, vocab=53)
    model, dec, w = build(rt, cfg, wdt_of(dtype), seed=16, max_tokens=4300)
    try:
        tok = C.tokens(cfg, 4200, 15)
        want = [0, 5, 3999, 4000, 4094, 4095, 4096, 4097, 4150, 4199]
        got = dec.step(tok, want)
        assert dec.pos == len(tok)
        if "ref" not in _LONG_REF:  # the same weights and tokens for both matrix types
            _LONG_REF["ref"] = R.forward(cfg, w, tok)[want]
        assert rel_err(got, _LONG_REF["ref"]).max() < tol(dtype)
    finally:
        dec.close()
        model.close()


def test_sequence_cannot_pass_max_tokens(rt):
    from yalm_amd import models as M

    model, dec, _ = build(rt, C.ONLY_WINDOW, M.F32, seed=13, max_tokens=16)
    try:
        dec.step(C.tokens(C.ONLY_WINDOW, 16, 0))
        with pytest.raises(rt.YalmError):
            dec.step([1])
    finally:
        dec.close()
        model.close()


def test_mixed_scores_over_a_long_key_row(rt):
    """kv_heads x dim above the MFMA attention's key size: portions of a bf16 model take the
    f32 FMA kernel, with the same results."""
    from yalm_amd import models as M

    cfg = C.config([("attention_2", C.chunk(heads=10, kv_heads=5, dim=128, vdim=8, size=50, rot_dims=64, scale=0.09), None)],
                   width=64, vocab=101)
    model, dec, w = build(rt, cfg, M.BF16, seed=18)
    try:
        tok = C.tokens(cfg, 120, 17)
        ref = R.forward(cfg, w, tok)
        assert rel_err(run_portions(dec, tok, [70, 3, 1, 1]), ref).max() < BF16_TOL
    finally:
        dec.close()
        model.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_runner(rt, tmp_path, dtype):
    """bin/trace_run on a checkpoint folder written here: two requests one after the other,
    in portions, the second on the decoder the first gave back."""
    from yalm_amd import layered as Ly
    from yalm_amd.yalmfile import write_yalm

    cfg = C.MIXED
    t = Ly.lenuzen_random_tensors(cfg, seed=16)
    mdir = tmp_path / "model"
    mdir.mkdir()
    (mdir / "config.json").write_text(json.dumps(cfg))
    write_yalm(str(mdir / "model.safetensors"), {k: Ly.f32_to_bf16(v).reshape(v.shape) for k, v in t.items()}, {},
               {k: "BF16" for k in t})
    a, b = C.tokens(cfg, 30, 12), C.tokens(cfg, 19, 13)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:20], "want": [19, 0, 7]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[20:22], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[22:], "want": [7]}], "end": ["a"]},
        {"step": 3, "entries": [{"id": "b", "tokens": b[:18], "want": [17]}], "end": []},
        {"step": 4, "entries": [{"id": "b", "tokens": b[18:], "want": [0]}], "end": ["b"]},
    ]
    out = tmp_path / "out"
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(mdir), "--dtype", dtype, "--out", str(out),
                        "--max-tokens", "64"], input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True,
                       text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done %d" % i for i in range(5)]
    assert not (out / "1.f32").exists()
    w = {k: v.astype(np.float64) for k, v in t.items()}
    ra, rb = R.forward(cfg, w, a), R.forward(cfg, w, b)
    lim = F32_TOL if dtype == "float32" else BF16_TOL
    V = cfg["vocab"]
    assert rel_err(np.fromfile(out / "0.f32", "<f4").reshape(-1, V), ra[[19, 0, 7]]).max() < lim
    assert rel_err(np.fromfile(out / "2.f32", "<f4").reshape(-1, V), ra[[29]]).max() < lim
    assert rel_err(np.fromfile(out / "3.f32", "<f4").reshape(-1, V), rb[[17]]).max() < lim
    assert rel_err(np.fromfile(out / "4.f32", "<f4").reshape(-1, V), rb[[18]]).max() < lim
