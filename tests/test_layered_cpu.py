"""CPU: configuration reading and weight packing of layer-list designs, and the plain
restatement's own consistency (no GPU here)."""
import numpy as np
import pytest

import sinulorn_cases as C
import sinulorn_ref as R
from yalm_amd import layered as Ly
from yalm_amd import models as M


def test_config_reads_every_size_and_constant():
    c = Ly.sinulorn_config(C.MIXED, max_tokens=300)
    assert (c.width, c.vocab, c.embed_scale, c.norm_eps, c.max_tokens) == (96, 211, 7.0, 1e-5, 300)
    l0, l1, l2, l3, l4, l5 = c.layers
    assert (l0.mixer, l0.heads, l0.kv_heads, l0.dim, l0.vdim, l0.conv, l0.ff_kind, l0.ff) == (
        Ly.MIX_DELTA, 4, 2, 24, 40, 4, Ly.FF_DENSE, 72)
    assert (l1.mixer, l1.kv_from, l1.kv_rank, l1.q_rank, l1.attn_scale) == (Ly.MIX_LATENT, -1, 40, 56, 0.3)
    assert (l1.experts, l1.top, l1.groups, l1.groups_keep, l1.router_scale, l1.limit, l1.shared_ff, l1.shared_limit) == (
        8, 2, 4, 2, 1.75, 1.5, 40, 0.75)
    assert (l2.mixer, l2.rec_width, l2.blocks, l2.conv, l2.ff_kind) == (Ly.MIX_RGLRU, 80, 5, 3, Ly.FF_NONE)
    assert l3.kv_from == 1 and l3.in_rows == l3.q_rank
    assert l4.shared_ff == 0 and l4.top == 1
    assert l0.in_rows == 2 * 2 * 24 + 2 * 4 * 40 + 2 * 4


def test_unknown_names_are_refused():
    bad = C.config([("sliding", {}, None)])
    with pytest.raises(ValueError):
        Ly.sinulorn_config(bad)


def test_pack_concatenates_transposes_and_stacks():
    cfg = C.MIXED
    t = Ly.sinulorn_random_tensors(cfg, seed=3)
    for wdt in (M.F32, M.BF16):
        c = Ly.sinulorn_config(cfg, weight_dtype=wdt)
        p = Ly.sinulorn_pack(c, t)
        f = (lambda a: a) if wdt == M.F32 else Ly.bf16_to_f32
        d0 = p["layers"][0]
        got = f(d0["w_in"])
        want = np.concatenate([t["l0.mix." + n] for n in ("q", "k", "v", "g", "b", "a")])
        assert np.array_equal(got, want)
        d1, l1 = p["layers"][1], c.layers[1]
        ukt = f(d1["w_ukt"])
        uk = t["l1.mix.uk"].reshape(l1.heads, l1.dim, l1.kv_rank)
        assert np.array_equal(ukt, uk.transpose(0, 2, 1))
        assert np.array_equal(f(d1["w_in"]), np.concatenate([t["l1.mix.dq"], t["l1.mix.dkv"]]))
        assert np.array_equal(f(d1["w_gate"])[5], t["l1.mlp.e5.gate"])
        assert np.array_equal(f(p["layers"][3]["w_in"]), t["l3.mix.dq"]) and "kv_norm" not in p["layers"][3]
        assert d1["router"].dtype == np.float32 and np.array_equal(d1["router"], t["l1.mlp.router"])
        d2 = p["layers"][2]
        assert np.array_equal(d2["in_bias"], np.concatenate([t["l2.mix.y.b"], t["l2.mix.x.b"]]))
        for l, d in zip(c.layers, p["layers"]):
            assert set(d) == set(Ly.packed_shapes(c, l))


def test_bf16_round_trip_is_nearest_even():
    x = np.array([1.0, 1.00390625, 1.01171875, -3.1415927, 1e-30], np.float32)
    b = Ly.f32_to_bf16(x)
    assert np.array_equal(Ly.bf16_to_f32(b)[:3], np.array([1.0, 1.0, 1.015625], np.float32))
    assert np.all(np.abs(Ly.bf16_to_f32(b) - x) <= np.abs(x) * 2.0**-8)


@pytest.mark.parametrize("cfg", [C.MIXED, C.ODD], ids=["mixed", "odd"])
def test_restatement_is_causal(cfg):
    """Position t of the plain restatement depends on positions 0..t only."""
    w = {k: v.astype(np.float64) for k, v in Ly.sinulorn_random_tensors(cfg, seed=1).items()}
    tok = C.tokens(cfg, 21)
    full = R.forward(cfg, w, tok)
    part = R.forward(cfg, w, tok[:9])
    assert np.allclose(full[:9], part, rtol=0, atol=1e-10)


def test_restatement_router_respects_groups():
    """An expert outside the kept groups is never chosen, however large its score."""
    rng = np.random.default_rng(0)
    E, G, keep, top, Wd = 8, 4, 1, 2, 12
    w = {"r.router": rng.standard_normal((E, Wd))}
    h = rng.standard_normal((50, Wd))
    idx, wt = R.route(w, "r.", h, {"experts": E, "top": top, "scale": 2.0, "groups": {"count": G, "keep": keep}})
    assert np.all(idx[:, 0] // (E // G) == idx[:, 1] // (E // G))
    z = h @ w["r.router"].T
    s = np.exp(z - z.max(1, keepdims=True))
    s /= s.sum(1, keepdims=True)
    assert np.array_equal(idx[:, 0], s.argmax(1))
    assert np.allclose(wt[:, 0], 2.0 * s.max(1))
