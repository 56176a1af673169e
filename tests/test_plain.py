"""Pins the plain implementation by what fixes it beside the reference's text: special
cases that reduce to a library routine, invariants, and vectors the reference's own tests
hold. Each check is chosen so that a plausible mistake fails it."""

from __future__ import annotations

import math

import numpy as np
import torch

from plain import llama_plain as P

LLAMA3 = dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=64)


def rnd(*shape, seed=0):
    return np.random.default_rng(seed).standard_normal(shape)


# ---------------------------------------------------------------- rms norm

def test_rmsnorm_unit_weight_is_x_over_rms():
    x = rnd(5, 48)
    got = P.rms_norm(x, np.ones(48), 1e-6)
    want = x / np.sqrt((x ** 2).mean(-1, keepdims=True) + 1e-6)
    np.testing.assert_allclose(got, want, rtol=1e-12)


def test_rmsnorm_scale_invariant_and_eps_inside_root():
    x = rnd(3, 32)
    w = 1 + 0.1 * rnd(32, seed=1)
    a, b = P.rms_norm(x, w, 0.0), P.rms_norm(1000 * x, w, 0.0)
    np.testing.assert_allclose(a, b, rtol=1e-10)
    # zero row: eps inside the root keeps it finite and zero
    z = P.rms_norm(np.zeros((1, 32)), w, 1e-5)
    assert np.all(z == 0)
    # tiny x: output = x / sqrt(eps) when mean square << eps (eps outside the root would give x/(rms+eps))
    t = np.full((1, 4), 1e-8)
    np.testing.assert_allclose(P.rms_norm(t, np.ones(4), 1e-4), t / math.sqrt(1e-16 + 1e-4), rtol=1e-9)


def test_rmsnorm_weight_is_applied():
    x = rnd(2, 16)
    w = np.arange(1, 17, dtype=float)
    np.testing.assert_allclose(P.rms_norm(x, w, 1e-6), w * P.rms_norm(x, np.ones(16), 1e-6), rtol=1e-12)


# -------------------------------------------------------------------- rope

def test_inv_freq_plain_formula():
    inv = P.rope_inv_freq(16, 10000.0, None)
    want = np.array([10000.0 ** (-2 * i / 16) for i in range(8)])
    np.testing.assert_allclose(inv, want, rtol=1e-6)


def test_llama3_factor_one_changes_nothing():
    s = dict(LLAMA3, factor=1.0)
    np.testing.assert_array_equal(P.rope_inv_freq(32, 500000.0, s), P.rope_inv_freq(32, 500000.0, None))


def test_llama3_bands():
    base = P.rope_inv_freq(32, 500000.0, None).astype(np.float64)
    got = P.rope_inv_freq(32, 500000.0, LLAMA3).astype(np.float64)
    wl = 2 * math.pi / base
    short, long_ = wl < 64 / 4.0, wl > 64 / 1.0
    mid = ~short & ~long_
    assert short.any() and long_.any() and mid.any()          # all three bands are non-empty
    np.testing.assert_allclose(got[short], base[short], rtol=1e-7)      # short waves untouched
    np.testing.assert_allclose(got[long_], base[long_] / 8.0, rtol=1e-6)  # long waves divided by factor
    assert np.all(got[mid] < base[mid]) and np.all(got[mid] > base[mid] / 8.0)  # a blend in between


def _pair_wavelengths(head_dim, theta):
    return 2 * math.pi * theta ** (np.arange(0, head_dim, 2) / head_dim)


def test_llama3_medium_band_falls_from_one_to_one_over_factor():
    """Several pairs inside the medium band: the ratio to the unscaled frequency is linear in
    old/wavelength, 1 at the short edge and 1/factor at the long edge, so it falls with the
    wavelength. A blend with ``smooth`` and ``1 - smooth`` swapped rises instead; one that
    interpolates in the wavelength rather than its inverse is not linear here."""
    d, theta = 64, 10000.0
    rule = dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=256)
    base = P.rope_inv_freq(d, theta, None).astype(np.float64)
    got = P.rope_inv_freq(d, theta, rule).astype(np.float64)
    wl = _pair_wavelengths(d, theta)
    mid = (wl >= 256 / 4.0) & (wl <= 256 / 1.0)
    assert mid.sum() >= 4
    ratio = got[mid] / base[mid]
    assert np.all(np.diff(ratio) < 0) and ratio[0] < 1.0 and ratio[-1] > 1 / 8.0
    # Written out independently of the blend: a line through (old/wl = high, 1) and (old/wl = low, 1/factor).
    x = 256.0 / wl[mid]
    line = 1 / 8.0 + (1 - 1 / 8.0) * (x - 1.0) / (4.0 - 1.0)
    np.testing.assert_allclose(ratio, line, rtol=2e-6)
    # One number by hand: halfway between the edges in old/wl (2.5) the ratio is (1 + 1/8) / 2.
    assert abs(np.interp(2.5, x[::-1], ratio[::-1]) - 0.5625) < 2e-3


def test_llama3_is_continuous_at_the_band_edges():
    """A pair whose wavelength sits exactly on an edge of the medium band gets what the band
    beyond that edge gets: unchanged at old/high, divided by the factor at old/low. The
    original length is chosen so that pair j lies on the edge."""
    d, theta, factor = 32, 500000.0, 8.0
    base = P.rope_inv_freq(d, theta, None).astype(np.float64)
    wl = 2 * math.pi / base
    j = 6
    for edge_factor, want in ((4.0, 1.0), (1.0, 1 / factor)):          # short edge: old/high; long edge: old/low
        for nudge in (1 - 1e-9, 1.0, 1 + 1e-9):                        # just inside, on, just outside the band
            rule = dict(factor=factor, low_freq_factor=1.0, high_freq_factor=4.0,
                        original_max_position_embeddings=edge_factor * wl[j] * nudge)
            got = float(P.rope_inv_freq(d, theta, rule)[j])
            assert abs(got / base[j] - want) < 1e-6, (edge_factor, nudge)


def test_rope_position_zero_is_identity_and_norms_are_kept():
    inv = P.rope_inv_freq(16, 10000.0, None)
    x = rnd(4, 3, 16)
    cos, sin = P.rope_cos_sin(np.zeros(4, dtype=np.int64), inv)
    np.testing.assert_allclose(P.apply_rope(x, cos, sin), x, atol=1e-15)
    cos, sin = P.rope_cos_sin(np.array([3, 50, 700, 1999]), inv)
    y = P.apply_rope(x, cos, sin)
    pair = lambda v: v[..., :8] ** 2 + v[..., 8:] ** 2          # pair (i, i + D/2)
    np.testing.assert_allclose(pair(y), pair(x), rtol=1e-9)


def test_rope_pairs_i_with_i_plus_half_not_neighbours():
    # A one-hot at dim 0 must spill into dim D/2 (rotate-half), not into dim 1 (interleaved).
    inv = P.rope_inv_freq(16, 10000.0, None)
    x = np.zeros((1, 1, 16)); x[0, 0, 0] = 1.0
    cos, sin = P.rope_cos_sin(np.array([1]), inv)
    y = P.apply_rope(x, cos, sin)[0, 0]
    assert abs(y[0] - math.cos(1.0)) < 1e-6 and abs(y[8] - math.sin(1.0)) < 1e-6
    assert np.all(np.abs(np.delete(y, [0, 8])) < 1e-12)


def test_rope_scores_depend_on_distance_only():
    inv = P.rope_inv_freq(32, 500000.0, LLAMA3)
    q, k = rnd(1, 1, 32, seed=3), rnd(1, 1, 32, seed=4)

    def score(m, n):
        cq, sq = P.rope_cos_sin(np.array([m]), inv)
        ck, sk = P.rope_cos_sin(np.array([n]), inv)
        return float((P.apply_rope(q, cq, sq) * P.apply_rope(k, ck, sk)).sum())

    assert abs(score(9, 4) - score(109, 104)) < 1e-4      # float32 angles: equal up to their rounding
    assert abs(score(9, 4) - score(4, 9)) > 1e-3          # and the sign of the distance matters


# --------------------------------------------------------------- attention

def test_attention_single_key_returns_its_value():
    q, k, v = rnd(1, 4, 16), rnd(1, 2, 16, seed=1), rnd(1, 2, 16, seed=2)
    out = P.causal_attention(q, k, v)
    for h in range(4):
        np.testing.assert_allclose(out[0, h], v[0, h // 2], rtol=1e-12)   # head h reads kv head h // group


def test_attention_zero_query_averages_visible_values():
    n = 6
    q, k, v = np.zeros((n, 2, 8)), rnd(n, 2, 8, seed=1), rnd(n, 2, 8, seed=2)
    out = P.causal_attention(q, k, v)
    for j in range(n):
        np.testing.assert_allclose(out[j], v[: j + 1].mean(0), rtol=1e-12)


def test_attention_equals_library_sdpa_with_causal_mask():
    n, hq, hkv, d = 23, 6, 2, 16
    q, k, v = rnd(n, hq, d), rnd(n, hkv, d, seed=1), rnd(n, hkv, d, seed=2)
    got = P.causal_attention(q, k, v)
    tq = torch.from_numpy(q).permute(1, 0, 2)[None]
    tk = torch.from_numpy(k).permute(1, 0, 2).repeat_interleave(hq // hkv, dim=0)[None]
    tv = torch.from_numpy(v).permute(1, 0, 2).repeat_interleave(hq // hkv, dim=0)[None]
    want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True)[0].permute(1, 0, 2).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-9, atol=1e-12)


def test_attention_is_causal():
    n = 9
    q, k, v = rnd(n, 2, 8), rnd(n, 2, 8, seed=1), rnd(n, 2, 8, seed=2)
    base = P.causal_attention(q, k, v)
    k2, v2 = k.copy(), v.copy()
    k2[5] += 3.0; v2[5] -= 2.0
    out = P.causal_attention(q, k2, v2)
    np.testing.assert_array_equal(out[:5], base[:5])
    assert np.abs(out[5:] - base[5:]).max() > 1e-3


def test_gqa_with_equal_heads_is_mha_and_window_keeps_recent_keys():
    n = 7
    q, k, v = rnd(n, 3, 8), rnd(n, 3, 8, seed=1), rnd(n, 3, 8, seed=2)
    out = P.causal_attention(q, k, v)
    for h in range(3):
        one = P.causal_attention(q[:, h:h + 1], k[:, h:h + 1], v[:, h:h + 1])
        np.testing.assert_allclose(out[:, h:h + 1], one, rtol=1e-12)
    w = P.causal_attention(q, k, v, window=1)
    np.testing.assert_allclose(w, v, rtol=1e-12)              # window 1: each token sees itself only


# ------------------------------------------------------------- feed-forward

def test_swiglu_against_library_silu_and_gate_up_order():
    x, wg, wu, wd = rnd(4, 8), rnd(12, 8, seed=1), rnd(12, 8, seed=2), rnd(8, 12, seed=3)
    got = P.swiglu_mlp(x, wg, wu, wd)
    tx = torch.from_numpy(x)
    want = (torch.nn.functional.silu(tx @ torch.from_numpy(wg).T) * (tx @ torch.from_numpy(wu).T)) @ torch.from_numpy(wd).T
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-10)
    assert np.abs(P.swiglu_mlp(x, wu, wg, wd) - got).max() > 1e-3   # gate and up are not interchangeable


# ------------------------------------------------------------------- model

def test_tied_head_equals_untied_copy_of_the_table(model_dirs, tmp_path):
    import json
    import shutil

    from plain.llama_plain import PlainLlama, read_safetensors
    from safetensors.numpy import save_file

    src = model_dirs["A"]                      # tied
    dst = tmp_path / "untied"
    dst.mkdir()
    cfg = json.loads((src / "config.json").read_text())
    cfg["tie_word_embeddings"] = False
    (dst / "config.json").write_text(json.dumps(cfg))
    w = read_safetensors(src / "model.safetensors")
    w["lm_head.weight"] = w["model.embed_tokens.weight"].copy()
    save_file({k: np.ascontiguousarray(v, dtype=np.float32) for k, v in w.items()}, str(dst / "model.safetensors"))
    toks = [5, 17, 3, 200, 41]
    np.testing.assert_allclose(PlainLlama(src).logits(toks), PlainLlama(dst).logits(toks), rtol=1e-12)
    shutil.rmtree(dst)


def test_a_layer_is_its_attention_half_followed_by_its_feed_forward_half(plain_models):
    """The arrangement of a layer, pinned by what each half reduces to. With the output
    projection zeroed a layer is h + mlp(norm2(h)); with the down projection zeroed it is
    h + attention(norm1(h)); and the full layer is the second applied to the result of the
    first. A feed-forward that reads the layer's input instead of the attention's result
    (a parallel block), a norm after the sum instead of before the part, or a missing
    residual path each break one of the three."""
    import copy

    m = plain_models["B"]
    c = m.cfg
    n = 21
    h = rnd(n, c.hidden, seed=8)
    cos, sin = P.rope_cos_sin(np.arange(n), m.inv_freq)
    pre = "model.layers.1."

    def variant(zeroed):
        v = copy.copy(m)
        v.w = dict(m.w)
        v.w[pre + zeroed] = np.zeros_like(m.w[pre + zeroed])
        return v

    only_ff = variant("self_attn.o_proj.weight").layer(1, h, cos, sin)
    want = h + P.swiglu_mlp(P.rms_norm(h, m.w[pre + "post_attention_layernorm.weight"], c.eps),
                            m.w[pre + "mlp.gate_proj.weight"], m.w[pre + "mlp.up_proj.weight"], m.w[pre + "mlp.down_proj.weight"])
    np.testing.assert_allclose(only_ff, want, rtol=1e-10, atol=1e-12)

    only_attn = variant("mlp.down_proj.weight").layer(1, h, cos, sin)
    x = P.rms_norm(h, m.w[pre + "input_layernorm.weight"], c.eps)
    q = P.apply_rope((x @ m.w[pre + "self_attn.q_proj.weight"].T).reshape(n, c.heads, c.head_dim), cos, sin)
    k = P.apply_rope((x @ m.w[pre + "self_attn.k_proj.weight"].T).reshape(n, c.kv_heads, c.head_dim), cos, sin)
    v = (x @ m.w[pre + "self_attn.v_proj.weight"].T).reshape(n, c.kv_heads, c.head_dim)
    want = h + P.causal_attention(q, k, v).reshape(n, -1) @ m.w[pre + "self_attn.o_proj.weight"].T
    np.testing.assert_allclose(only_attn, want, rtol=1e-10, atol=1e-12)
    assert np.abs(only_attn - h).max() > 1e-3 and np.abs(only_ff - h).max() > 1e-3

    full = m.layer(1, h, cos, sin)
    np.testing.assert_allclose(full, variant("self_attn.o_proj.weight").layer(1, only_attn, cos, sin), rtol=1e-10, atol=1e-12)
    parallel = only_attn + only_ff - h
    assert np.abs(full - parallel).max() > 1e-4


def test_logits_do_not_depend_on_a_shift_of_all_positions(plain_models):
    # Only distances count. A rotation applied with the wrong sign to k, or positions fed
    # to q only, breaks this. Float32 angles bound the agreement.
    m = plain_models["B"]
    toks = list(np.random.default_rng(5).integers(0, 512, 40))
    a, b = m.logits(toks, 0), m.logits(toks, 37)
    assert np.abs(a - b).max() / np.abs(a).max() < 2e-5


def test_logits_are_causal(plain_models):
    m = plain_models["A"]
    toks = list(np.random.default_rng(6).integers(0, 256, 30))
    a = m.logits(toks)
    toks2 = list(toks); toks2[20] = (toks2[20] + 1) % 256
    b = m.logits(toks2)
    np.testing.assert_array_equal(a[:20], b[:20])
    assert np.abs(a[20:] - b[20:]).max() > 1e-4


def test_norm_weights_matter(plain_models, model_dirs):
    # Random norm weights are 1 + N(0, 0.1): a forgotten multiply is visible.
    w = P.read_safetensors(model_dirs["A"] / "model.safetensors")
    nw = w["model.layers.0.input_layernorm.weight"]
    assert np.abs(nw - 1).max() > 0.05


def test_the_final_norm_stands_in_front_of_the_output_matrix(plain_models, model_dirs, tmp_path):
    """logits = head . (norm.weight * h / rms(h)) (prefixserve/model/llama.py:123-126). A model
    whose final norm weight is zero gives zero logits; doubling the weight doubles them; and a
    last hidden state scaled by 1,000 gives the same logits, because the norm divides the scale
    out. A ``logits()`` that skips the norm, applies it after the product or leaves out its
    weight fails one of the three."""
    import shutil

    from safetensors.numpy import save_file

    name = "B"
    toks = np.random.default_rng(3).integers(0, 512, 20).tolist()
    base = plain_models[name].logits(toks)
    w = P.read_safetensors(model_dirs[name] / "model.safetensors")

    def variant(folder, **changed):
        folder.mkdir()
        shutil.copy(model_dirs[name] / "config.json", folder / "config.json")
        save_file({k: np.ascontiguousarray(changed.get(k, v), dtype=np.float32) for k, v in w.items()},
                  str(folder / "model.safetensors"))
        return P.PlainLlama(folder)

    zero = variant(tmp_path / "zero", **{"model.norm.weight": np.zeros_like(w["model.norm.weight"])})
    assert np.abs(base).max() > 0.1 and np.array_equal(zero.logits(toks), np.zeros_like(base))
    twice = variant(tmp_path / "twice", **{"model.norm.weight": 2.0 * w["model.norm.weight"]})
    assert np.allclose(twice.logits(toks), 2.0 * base, rtol=1e-12, atol=0)
    # Scale what the last layer adds to the residual stream: its down projection. With a tiny
    # eps the norm removes almost all of it; a product without the norm would grow with it.
    plain = plain_models[name]
    h = plain.hidden(toks)
    head = plain.w["lm_head.weight"]
    by_hand = P.rms_norm(h, plain.w["model.norm.weight"], plain.cfg.eps) @ head.T
    assert np.allclose(base, by_hand, rtol=1e-12, atol=1e-12)
    assert np.allclose(P.rms_norm(1000.0 * h, plain.w["model.norm.weight"], plain.cfg.eps) @ head.T, base, rtol=1e-6)
    assert not np.allclose(h @ head.T, base, rtol=0.05, atol=0.05 * np.abs(base).max())


def test_bf16_reader_is_exact():
    from safetensors.torch import save_file
    import tempfile, os

    t = torch.randn(7, 5).to(torch.bfloat16)
    with tempfile.TemporaryDirectory() as d:
        save_file({"x": t}, os.path.join(d, "m.safetensors"))
        got = P.read_safetensors(os.path.join(d, "m.safetensors"))["x"]
    np.testing.assert_array_equal(got, t.float().numpy())


# ---------------------------------------------------------------- sampling

def test_plain_sampler():
    logits = np.array([0.0, 1.0, 3.0, 3.0, -2.0])
    assert P.sample_plain(logits, 0.0, 0.3) == 2                       # lowest index among equal maxima
    p = np.exp(logits / 0.7); p /= p.sum()
    edges = np.cumsum(p)
    assert P.sample_plain(logits, 0.7, edges[1] - 1e-9) == 1 and P.sample_plain(logits, 0.7, edges[1] + 1e-9) == 2
    us = [P.uniform_for(3, 99, i) for i in range(2000)]
    assert 0 <= min(us) and max(us) < 1 and abs(np.mean(us) - 0.5) < 0.03
    assert P.uniform_for(3, 99, 5) == P.uniform_for(3, 99, 5) != P.uniform_for(3, 98, 5)
