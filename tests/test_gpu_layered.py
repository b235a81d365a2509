"""MI355X: the layer-list engine (Sinulorn) against the plain float64 restatement in
tests/sinulorn_ref.py, on small random models made here.

Errors are per position: || got - ref || / || ref || over the vocabulary. With f32 matrices
the engine differs from the restatement by f32 rounding only (F32_TOL); with bf16 matrices
by the rounding of weights' products' inputs (BF16_TOL). A lost key, a stale state or a
token one place off moves the logits by orders of magnitude more than F32_TOL.
"""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import sinulorn_cases as C
import sinulorn_ref as R

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F32_TOL, BF16_TOL = 2e-4, 6e-2


@pytest.fixture(scope="module")
def rt():
    from yalm_amd import runtime

    runtime.check(runtime.lib.yalm_set_device(0))
    return runtime


def build(rt, cfg, wdt, seed=0, max_tokens=512):
    from yalm_amd import layered as Ly

    t = Ly.sinulorn_random_tensors(cfg, seed=seed)
    c = Ly.sinulorn_config(cfg, max_tokens=max_tokens, weight_dtype=wdt)
    model = rt.SeqModel.from_packed(c, Ly.sinulorn_pack(c, t))
    return model, rt.SeqDecoder(model), {k: v.astype(np.float64) for k, v in t.items()}


def rel_err(got, ref):
    return np.linalg.norm(got - ref, axis=-1) / np.linalg.norm(ref, axis=-1)


def close_enough(got, ref, dtype, frac=1.0):
    """f32: every position within F32_TOL. bf16: every position within BF16_TOL, except
    that models with routed experts may miss it at a share 1 - frac of the positions: a
    router's near tie resolved the other way by the rounding of an earlier product moves
    that token's (and, through recurrent layers, some later tokens') logits far more than
    rounding does."""
    e = rel_err(got, ref)
    if dtype == "f32":
        return e.max() < F32_TOL
    return np.mean(e < BF16_TOL) >= frac


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


ALONE = {"latent": C.ONLY_LATENT, "rglru": C.ONLY_RGLRU, "delta": C.ONLY_DELTA, "dense": C.ONLY_DENSE, "moe": C.ONLY_MOE}


@pytest.mark.parametrize("name", sorted(ALONE))
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_each_mechanism_alone(rt, name, dtype):
    """One-layer models: a whole prompt that spans more than one GEMM tile and key tile."""
    from yalm_amd import models as M

    cfg = ALONE[name]
    model, dec, w = build(rt, cfg, M.F32 if dtype == "f32" else M.BF16, seed=2)
    try:
        tok = C.tokens(cfg, 150, 1)
        got = dec.step(tok, list(range(len(tok))))
        ref = R.forward(cfg, w, tok)
        assert close_enough(got, ref, dtype, 0.95 if name == "moe" else 1.0)
    finally:
        dec.close()
        model.close()


@pytest.mark.parametrize("cfg", [C.MIXED, C.ODD, C.WIDE], ids=["mixed", "odd", "wide"])
def test_residual_stream_after_every_layer(rt, cfg):
    from yalm_amd import models as M

    model, dec, w = build(rt, cfg, M.F32, seed=4)
    try:
        tok = C.tokens(cfg, 33, 2)
        dec.layer_dump(True)
        dec.step(tok)
        got = dec.get_layers(len(tok))
        ref = []
        R.forward(cfg, w, tok, ref)
        for i, r in enumerate(ref):
            assert rel_err(got[i], r).max() < 5e-5, f"layer {i} ({cfg['layers'][i]['type']})"
    finally:
        dec.close()
        model.close()


@pytest.mark.parametrize("cfg", [C.MIXED, C.ODD, C.WIDE], ids=["mixed", "odd", "wide"])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_prefill_then_token_by_token(rt, cfg, dtype):
    """A prompt in one step, then single tokens through the caches and states."""
    from yalm_amd import models as M

    model, dec, w = build(rt, cfg, M.F32 if dtype == "f32" else M.BF16, seed=5)
    try:
        tok = C.tokens(cfg, 37 + 40, 3)
        got = run_portions(dec, tok, [37] + [1] * 40)
        ref = R.forward(cfg, w, tok)
        assert close_enough(got, ref, dtype, 0.6)
        assert dec.pos == len(tok)
    finally:
        dec.close()
        model.close()


# portions down to two tokens, across the single-token kernels' limit of 8 rows (8 | 9),
# the GEMM's 64-row tiles (64 | 65), the attention's 64-key tiles and 16-row blocks
PORTIONS = [
    [2, 2, 3, 1, 9, 8, 64, 65, 2, 1, 1, 63],
    [1, 1, 1, 2, 128, 3, 16, 17, 15],
    [200, 2, 9],
    [7, 57, 1, 64, 1, 2, 2, 2],
]


@pytest.mark.parametrize("cfg", [C.MIXED, C.ODD], ids=["mixed", "odd"])
@pytest.mark.parametrize("sizes", PORTIONS, ids=[str(i) for i in range(len(PORTIONS))])
def test_portions_of_any_size(rt, cfg, sizes):
    from yalm_amd import models as M

    model, dec, w = build(rt, cfg, M.F32, seed=6)
    try:
        tok = C.tokens(cfg, 260, 4)
        ref = R.forward(cfg, w, tok)
        got = run_portions(dec, tok, sizes)
        assert rel_err(got, ref).max() < F32_TOL
        dec.reset()
        whole = dec.step(tok, list(range(len(tok))))
        assert rel_err(got, whole).max() < 5e-5  # the cut changes the rounding only
    finally:
        dec.close()
        model.close()


def test_bf16_stack_without_routing_is_strict(rt):
    """Every mixer in bf16 with dense feed-forwards: no routing tie can excuse a position."""
    from yalm_amd import models as M

    cfg = C.MIXED_DENSE
    model, dec, w = build(rt, cfg, M.BF16, seed=15)
    try:
        tok = C.tokens(cfg, 180, 14)
        ref = R.forward(cfg, w, tok)
        assert rel_err(dec.step(tok, list(range(len(tok)))), ref).max() < BF16_TOL
        dec.reset()
        assert rel_err(run_portions(dec, tok, [2, 70, 1, 1, 9, 3] + [1] * 20), ref).max() < BF16_TOL
    finally:
        dec.close()
        model.close()


def test_large_tile_products_bf16(rt):
    """Tile-aligned sizes and a portion of more than 256 tokens: the plain products (input and
    output projections with and without bias, the feed-forward's down projection, the head)
    take the prefill unit's large-tile GEMM in its bf16 instantiation; shorter portions and
    single tokens of the same sequence take the general kernels."""
    from yalm_amd import models as M

    cfg = C.TILED
    model, dec, w = build(rt, cfg, M.BF16, seed=18, max_tokens=700)
    try:
        tok = C.tokens(cfg, 600, 18)
        ref = R.forward(cfg, w, tok)
        assert rel_err(dec.step(tok, list(range(len(tok)))), ref).max() < BF16_TOL
        dec.reset()
        assert rel_err(run_portions(dec, tok, [300, 5, 1, 1, 257, 20]), ref).max() < BF16_TOL
    finally:
        dec.close()
        model.close()


def test_large_tile_clamped_pair_bf16(rt):
    """The shared expert's clamped gated pair through the large-tile GEMM."""
    from yalm_amd import models as M

    cfg = C.TILED_MOE
    model, dec, w = build(rt, cfg, M.BF16, seed=19, max_tokens=400)
    try:
        tok = C.tokens(cfg, 320, 19)
        assert close_enough(dec.step(tok, list(range(len(tok)))), R.forward(cfg, w, tok), "bf16", 0.95)
    finally:
        dec.close()
        model.close()


def test_portions_bf16_differ_by_rounding_only(rt):
    from yalm_amd import models as M

    model, dec, w = build(rt, C.WIDE, M.BF16, seed=7)
    try:
        tok = C.tokens(C.WIDE, 200, 5)
        whole = dec.step(tok, list(range(len(tok))))
        dec.reset()
        got = run_portions(dec, tok, [3, 70, 2, 1, 1, 9, 50])
        assert close_enough(got, whole, "bf16", 0.9)  # WIDE routes in its last layer only
        assert close_enough(got, R.forward(C.WIDE, w, tok), "bf16", 0.9)
    finally:
        dec.close()
        model.close()


def test_decoder_reused_after_reset(rt):
    """States of an ended sequence must not leak into the next one: the second sequence on
    a reused decoder equals the same sequence on a fresh decoder bit for bit."""
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
    """Two decoders on one model, their steps interleaved: each equals its sequence alone."""
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


def test_far_keys_decide_the_output(rt):
    """Peaked attention over a long prompt. The restatement's own softmax weights name a
    late query whose winning key lies more than 200 positions back; changing THAT token must
    move the query's logits, and the engine must follow, with the query inside a prompt's
    portion and decoded alone."""
    from yalm_amd import models as M

    cfg = C.config([("latent_attention", C.latent(heads=2, dim=16, vdim=24, kv_rank=40, q_rank=24, scale=1.5), None)],
                   width=64, vocab=101)
    model, dec, w = build(rt, cfg, M.F32, seed=9, max_tokens=600)
    try:
        a = C.tokens(cfg, 450, 8)
        eps, m = cfg["norm"]["eps"], cfg["layers"][0]["mixer"]
        h = R.rms_norm(R.embed(cfg, w, a), w["l0.norm1"], eps)
        P = R.attention_weights(cfg, w, "l0.mix.", h, m, eps, R.latent(cfg, w, "l0.mix.", h, m, eps))
        far = [(P[hh, t].max(), t, int(P[hh, t].argmax())) for hh in range(2) for t in range(300, 450)
               if t - int(P[hh, t].argmax()) >= 200]
        assert far, "no late query with a far winning key: pick another seed"
        weight, t, j = max(far)
        assert weight > 0.5
        b = list(a)
        b[j] = (b[j] + 17) % cfg["vocab"]
        ra, rb = R.forward(cfg, w, a), R.forward(cfg, w, b)
        assert rel_err(ra[t], rb[t]) > 100 * F32_TOL  # the far key decides position t
        for tok, ref in ((a, ra), (b, rb)):
            for sizes in ([440], [t] + [1] * 5):  # t in a prompt's portion / decoded alone
                dec.reset()
                got = run_portions(dec, tok, sizes)
                assert rel_err(got, ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


@pytest.mark.parametrize("n", [1, 2, 3, 5])
def test_first_tokens(rt, n):
    """Sequences shorter than the convolutions' taps: zeros before the start, states from zero."""
    from yalm_amd import models as M

    cfg = C.MIXED
    model, dec, w = build(rt, cfg, M.F32, seed=10)
    try:
        tok = C.tokens(cfg, n, 9)
        ref = R.forward(cfg, w, tok)
        assert rel_err(dec.step(tok, list(range(n))), ref).max() < F32_TOL
        dec.reset()
        assert rel_err(run_portions(dec, tok, [1] * n), ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_long_decoding(rt):
    from yalm_amd import models as M

    cfg = C.ODD
    model, dec, w = build(rt, cfg, M.F32, seed=11)
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
    model, dec, w = build(rt, cfg, M.F32, seed=12)
    try:
        prompt = C.tokens(cfg, 12, 11)
        dec.step(prompt[:-1])
        gen = dec.generate_greedy(prompt[-1], 24)
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


def test_prompt_longer_than_one_internal_portion(rt):
    """A step of more tokens than the engine's work buffers hold (4096) is cut inside the
    engine; asked rows on both sides of the cut come back in order."""
    from yalm_amd import models as M

    cfg = C.config([("rglru", C.rglru(width=24, blocks=3, conv=3), None),
                    ("latent_attention", C.latent(heads=1, dim=8, vdim=8, kv_rank=16, q_rank=8, scale=0.35), None)],
                   width=32, vocab=53)
    model, dec, w = build(rt, cfg, M.F32, seed=16, max_tokens=4300)
    try:
        tok = C.tokens(cfg, 4200, 15)
        want = [0, 5, 4094, 4095, 4096, 4097, 4150, 4199]
        got = dec.step(tok, want)
        assert dec.pos == len(tok)
        ref = R.forward(cfg, w, tok)[want]
        assert rel_err(got, ref).max() < F32_TOL
    finally:
        dec.close()
        model.close()


def test_greedy_graph_replays_match_eager_steps(rt):
    """The greedy loop replays one captured token graph. Several generate calls with ordinary
    (eager) steps and synchronisations between them: every replayed token equals the argmax of
    an eager step of a second decoder fed the same tokens."""
    from yalm_amd import models as M

    cfg = C.MIXED
    model, dec, w = build(rt, cfg, M.F32, seed=17)
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
            extra = C.tokens(cfg, 2, 17 + n)  # eager work on both between the replays
            a = dec.step(extra, [1])
            b = eager.step(extra, [1])
            assert np.array_equal(a, b)
            tok = int(np.argmax(a[0]))
        assert dec.pos == eager.pos
    finally:
        dec.close()
        eager.close()
        model.close()


def test_sequence_cannot_pass_max_tokens(rt):
    from yalm_amd import models as M

    model, dec, _ = build(rt, C.ONLY_RGLRU, M.F32, seed=13, max_tokens=16)
    try:
        dec.step(C.tokens(C.ONLY_RGLRU, 16, 0))
        with pytest.raises(rt.YalmError):
            dec.step([1])
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
    t = Ly.sinulorn_random_tensors(cfg, seed=14)
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
    tol = F32_TOL if dtype == "float32" else 4 * BF16_TOL  # bf16: a handful of rows, routing ties included
    V = cfg["vocab"]
    g0 = np.fromfile(out / "0.f32", "<f4").reshape(-1, V)
    assert rel_err(g0, ra[[19, 0, 7]]).max() < tol
    assert rel_err(np.fromfile(out / "2.f32", "<f4").reshape(-1, V), ra[[29]]).max() < tol
    assert rel_err(np.fromfile(out / "3.f32", "<f4").reshape(-1, V), rb[[17]]).max() < tol
    assert rel_err(np.fromfile(out / "4.f32", "<f4").reshape(-1, V), rb[[18]]).max() < tol
