"""Pins the plain implementation by what fixes it beside the reference's text: vectors the
reference's own tests hold, special cases that reduce to a library routine, invariants.
Each is chosen so that a plausible mistake fails it."""
import math

import numpy as np
import pytest
import torch

import plain_model as pm


# ---- vectors held by the reference's tests (tests/Daisi.Llogos.Tests/Cpu/MathOpsTests.cs) ----
def test_linear_layout_vector():
    # MathOpsTests.cs:10-28: W is [out, in]; a transposed reading gives other numbers
    a = np.array([[1, 2, 3], [4, 5, 6]], dtype=float)
    w = np.array([[7, 9, 11], [8, 10, 12]], dtype=float)
    assert np.allclose(pm.linear(a, w), [[58, 64], [139, 154]])


def test_linear_identity_and_bias():
    x = np.arange(9, dtype=float).reshape(3, 3)
    assert np.allclose(pm.linear(x, np.eye(3)), x)                      # MathOpsTests.cs:31-46
    assert np.allclose(pm.linear(x, np.eye(3), np.array([1., 2., 3.])), x + [1, 2, 3])


def test_rms_norm_vectors():
    # MathOpsTests.cs:129-169
    out = pm.rms_norm(np.array([1., 2., 3., 4.]), np.ones(4), 1e-6)
    assert np.allclose(out, np.array([1., 2., 3., 4.]) / math.sqrt(7.5 + 1e-6))
    out = pm.rms_norm(np.array([2., 2., 2., 2.]), np.array([.5, 1., 1.5, 2.]), 1e-6)
    assert np.allclose(out, [.5, 1., 1.5, 2.], atol=1e-6)


def test_rms_norm_eps_inside_root_and_plain_weight():
    # eps outside the root or a (1 + w) weight would change these
    assert np.all(pm.rms_norm(np.zeros(8), np.ones(8), 1e-5) == 0)
    x = np.full(4, 1e-3)
    assert np.allclose(pm.rms_norm(x, np.ones(4), 1e-2), x / math.sqrt(1e-6 + 1e-2))
    assert np.allclose(pm.rms_norm(np.ones(4), np.zeros(4), 1e-6), 0)


def test_silu_vectors():
    # MathOpsTests.cs:260-304
    z = np.array([-2., -1., 0., 1., 2.])
    assert np.allclose(pm.silu(z), z / (1 + np.exp(-z)))
    assert pm.silu(np.array([0.]))[0] == 0
    assert abs(pm.silu(np.array([10.]))[0] - 10) < 0.01
    assert np.allclose(pm.silu(z) - pm.silu(-z), z)                     # odd part is the identity


def test_softmax_vectors():
    # MathOpsTests.cs:186-243
    assert np.allclose(pm.softmax(np.zeros(5)), 0.2)
    p = pm.softmax(np.array([100., 200., 300.]))
    assert np.isfinite(p).all() and abs(p.sum() - 1) < 1e-12 and p[2] > p[1] > p[0]


def test_rope_vectors():
    # MathOpsTests.cs:321-384: position 0 is the identity, the norm is kept
    f = pm.rope_frequencies(4, 10000.0)
    q = np.array([[1., 2., 3., 4.]])
    for fn in (pm.rope_split_half, pm.rope_interleaved):
        assert np.allclose(fn(q, [0], 1, 4, f), q)
        r = fn(q, [42], 1, 4, f)
        assert abs(np.linalg.norm(r) - np.linalg.norm(q)) < 1e-9
        assert not np.allclose(fn(np.array([[1., 0, 0, 0, 0, 1., 0, 0]]), [5], 2, 4, f)[0, 0], 1.0)


# ---- special cases that reduce to a library routine ----
def test_rope_is_a_complex_multiplication():
    rng = np.random.default_rng(0)
    hd, pos = 16, 37
    f = pm.rope_frequencies(hd, 1e4)
    x = rng.standard_normal((1, hd))
    z = (x[0, :hd // 2] + 1j * x[0, hd // 2:]) * np.exp(1j * pos * f)   # a wrong sign of sin fails here
    r = pm.rope_split_half(x, [pos], 1, hd, f)[0]
    assert np.allclose(r[:hd // 2], z.real) and np.allclose(r[hd // 2:], z.imag)
    assert np.allclose(f, 1e4 ** (-np.arange(0, hd, 2) / hd))


def test_rope_pairings_agree_under_row_permutation():
    # interleaved on permuted rows == split-half on the original rows (Rope.cs:65-76)
    rng = np.random.default_rng(1)
    hd, heads, t = 8, 2, 5
    x = rng.standard_normal((t, heads * hd))
    f = pm.rope_frequencies(hd, 1e4)
    perm = np.concatenate([np.arange(0, hd, 2), np.arange(1, hd, 2)])   # interleaved -> halves
    xs = x.reshape(t, heads, hd)[:, :, perm].reshape(t, -1)
    a = pm.rope_interleaved(x, range(t), heads, hd, f).reshape(t, heads, hd)[:, :, perm].reshape(t, -1)
    b = pm.rope_split_half(xs, range(t), heads, hd, f)
    assert np.allclose(a, b)


def test_rope_partial_rotation_leaves_the_rest():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((3, 16))
    f = pm.rope_frequencies(8, 1e4)                                      # rotate 8 of 16
    r = pm.rope_split_half(x, [3, 4, 5], 1, 16, f)
    assert np.allclose(r[:, 8:], x[:, 8:]) and not np.allclose(r[:, :8], x[:, :8])


def test_rope_scores_depend_on_distance_only():
    rng = np.random.default_rng(3)
    hd = 32
    f = pm.rope_frequencies(hd, 5e5)
    q, k = rng.standard_normal((1, hd)), rng.standard_normal((1, hd))
    def score(m, n):
        return (pm.rope_split_half(q, [m], 1, hd, f) @ pm.rope_split_half(k, [n], 1, hd, f).T).item()
    assert abs(score(10, 3) - score(110, 103)) < 1e-9
    assert abs(score(10, 3) - score(3, 10)) > 1e-6                      # and on its sign


def test_llama3_factors():
    f = pm.rope_frequencies(64, 5e5)
    fac = pm.llama3_frequency_factors(f, 8.0, 1.0, 4.0, 8192)
    assert np.all(np.diff(fac) >= 0) and fac[0] == 1.0 and fac[-1] == 8.0
    wl = 2 * math.pi / f
    assert np.all(fac[wl < 8192 / 4] == 1.0) and np.all(fac[wl > 8192] == 8.0)
    mid = (wl >= 8192 / 4) & (wl <= 8192)
    assert mid.any() and np.all((fac[mid] >= 1.0) & (fac[mid] <= 8.0))
    assert np.allclose(pm.llama3_frequency_factors(f, 1.0, 1.0, 4.0, 8192), 1.0)


def test_llama3_band_mixes_frequencies_not_divisors():
    """Numbers worked by hand.  original 8192, low 1, high 4, factor 8: a pair that turns 2.5
    times in the original context is half way through the band, so its frequency becomes
    f * (0.5 / 8 + 0.5) = 0.5625 f and its divisor 16 / 9.  Mixing the divisors (0.5 * 8 +
    0.5 * 1 = 4.5), a band mixed the other way round (1 / (0.5 + 0.5 / 8) is the same at the
    middle, so a second point at a quarter of the band separates that), or wavelength and
    frequency taken for one another would all give other numbers."""
    f_of = lambda turns: np.array([turns * 2.0 * math.pi / 8192.0])
    assert pm.llama3_frequency_factors(f_of(2.5), 8.0, 1.0, 4.0, 8192)[0] == pytest.approx(16.0 / 9.0, rel=1e-12)
    # a quarter of the way (1.75 turns): f * (0.75 / 8 + 0.25) = 0.34375 f -> divisor 32 / 11
    assert pm.llama3_frequency_factors(f_of(1.75), 8.0, 1.0, 4.0, 8192)[0] == pytest.approx(32.0 / 11.0, rel=1e-12)
    # the band's ends meet the flat parts: no jump
    assert pm.llama3_frequency_factors(f_of(4.0), 8.0, 1.0, 4.0, 8192)[0] == pytest.approx(1.0, rel=1e-12)
    assert pm.llama3_frequency_factors(f_of(1.0), 8.0, 1.0, 4.0, 8192)[0] == pytest.approx(8.0, rel=1e-12)
    # other constants: original 64, low 2, high 6, factor 3; 3 turns are a quarter of the band:
    # f * (0.75 / 3 + 0.25) = 0.5 f
    f = np.array([3 * 2.0 * math.pi / 64.0])
    assert pm.llama3_frequency_factors(f, 3.0, 2.0, 6.0, 64)[0] == pytest.approx(2.0, rel=1e-12)


def test_per_head_norm_is_rms_norm_head_by_head_with_one_weight():
    """Daisi.Llogos.Cpu/CpuBackend.cs:406-421: every head's head_dim values are normed on
    their own, all heads with the same [head_dim] weight.  A norm over the whole row, a weight
    per head, or eps taken per row would all fail one of these."""
    rng = np.random.default_rng(5)
    t, n_heads, hd, eps = 3, 4, 8, 1e-3
    x = rng.standard_normal((t, n_heads * hd)) * np.repeat([0.01, 1.0, 30.0, 0.3], hd)   # heads of unlike size
    w = rng.standard_normal(hd)
    got = pm.per_head_rms_norm(x, w, n_heads, hd, eps)
    for h in range(n_heads):
        assert np.allclose(got[:, h * hd:(h + 1) * hd], pm.rms_norm(x[:, h * hd:(h + 1) * hd], w, eps), rtol=1e-13)
    whole = pm.rms_norm(x, np.tile(w, n_heads), eps)
    assert not np.allclose(got, whole, rtol=1e-2)
    # eps counts per head: the small head is damped by it, the large ones are not
    small = got[:, :hd] / w
    assert np.all(np.abs((small * small).mean(-1) - 1.0) > 0.5)
    big = got[:, 2 * hd:3 * hd] / w
    assert np.allclose((big * big).mean(-1), 1.0, atol=1e-4)
    # one head is the plain norm; one kv head (MQA) the same
    assert np.allclose(pm.per_head_rms_norm(x[:, :hd], w, 1, hd, eps), pm.rms_norm(x[:, :hd], w, eps), rtol=1e-13)
    # a row's result does not depend on the other rows
    assert np.allclose(pm.per_head_rms_norm(x[1:2], w, n_heads, hd, eps), got[1:2], rtol=1e-13)


def test_linear_scaling_stretches_positions():
    """rope_scaling 'linear' with factor s: position s * p of the scaled model is position p of
    the unscaled one; unknown kinds are refused."""
    base = dict(vocab_size=50, hidden_size=32, intermediate_size=48, num_hidden_layers=1, num_attention_heads=2,
                head_dim=16, rope_theta=1e4)
    plain_f = pm.PlainConfig(dict(base, architectures=["LlamaForCausalLM"])).frequencies()
    scaled = pm.PlainConfig(dict(base, architectures=["LlamaForCausalLM"], rope_scaling={"rope_type": "linear", "factor": 4.0}))
    assert np.allclose(scaled.frequencies(), plain_f / 4.0, rtol=1e-15)
    x = np.random.default_rng(0).standard_normal((3, 32))
    a = pm.rope_split_half(x, [0, 8, 20], 2, 16, scaled.frequencies())
    b = pm.rope_split_half(x, [0, 2, 5], 2, 16, plain_f)
    assert np.allclose(a, b, atol=1e-12)
    with pytest.raises(ValueError, match="yarn"):
        pm.PlainConfig(dict(base, architectures=["LlamaForCausalLM"], rope_scaling={"rope_type": "yarn", "factor": 2.0})).frequencies()


def _sdpa(q, k, v, n_heads, n_kv, hd, causal=True):
    t = q.shape[0]
    qt = torch.tensor(q).reshape(t, n_heads, hd).transpose(0, 1)
    kt = torch.tensor(k).reshape(t, n_kv, hd).transpose(0, 1).repeat_interleave(n_heads // n_kv, dim=0)
    vt = torch.tensor(v).reshape(t, n_kv, hd).transpose(0, 1).repeat_interleave(n_heads // n_kv, dim=0)
    o = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, is_causal=causal)
    return o.transpose(0, 1).reshape(t, n_heads * hd).numpy()


@pytest.mark.parametrize("n_heads,n_kv", [(4, 4), (4, 2), (6, 1), (1, 1)])
def test_attention_against_library(n_heads, n_kv):
    rng = np.random.default_rng(4)
    t, hd = 9, 8
    q = rng.standard_normal((t, n_heads * hd))
    k = rng.standard_normal((t, n_kv * hd))
    v = rng.standard_normal((t, n_kv * hd))
    assert np.allclose(pm.attention(q, k, v, n_heads, n_kv, hd), _sdpa(q, k, v, n_heads, n_kv, hd), atol=1e-10)


def test_attention_special_cases():
    rng = np.random.default_rng(5)
    t, hd = 6, 4
    q, k, v = (rng.standard_normal((t, hd)) for _ in range(3))
    o = pm.attention(q, k, v, 1, 1, hd)
    assert np.allclose(o[0], v[0])                                       # one visible key: its value
    o = pm.attention(np.zeros((t, hd)), k, v, 1, 1, hd)
    assert np.allclose(o[3], v[:4].mean(0))                              # equal scores: the mean
    # the group of a head is head // (heads / kv heads), not head % kv heads
    q2 = rng.standard_normal((t, 4 * hd)); k2 = rng.standard_normal((t, 2 * hd)); v2 = rng.standard_normal((t, 2 * hd))
    o2 = pm.attention(q2, k2, v2, 4, 2, hd)
    h1 = pm.attention(q2[:, hd:2 * hd], k2[:, :hd], v2[:, :hd], 1, 1, hd)
    assert np.allclose(o2[:, hd:2 * hd], h1)


def test_attention_window_and_sinks():
    rng = np.random.default_rng(6)
    t, hd = 12, 4
    q, k, v = (rng.standard_normal((t, hd)) for _ in range(3))
    full = pm.attention(q, k, v, 1, 1, hd)
    win = pm.attention(q, k, v, 1, 1, hd, window=4)
    assert np.allclose(win[:4], full[:4]) and not np.allclose(win[8], full[8])
    assert np.allclose(win[8], pm.attention(q[5:9], k[5:9], v[5:9], 1, 1, hd)[-1])   # exactly the last 4 keys
    snk = pm.attention(q, k, v, 1, 1, hd, window=4, sinks=2)
    idx = [0, 1, 7, 8, 9, 10]
    s = (k[idx] @ q[10]) / math.sqrt(hd)
    assert np.allclose(snk[10], pm.softmax(s) @ v[idx])
    assert pm.visible(10, 6, 4, 0) is False and pm.visible(10, 7, 4, 0) is True and pm.visible(5, 6) is False


# ---- the whole model ----
def _tiny(tmp_path, cfg, llogos, seed=3):
    folder = str(tmp_path / "m")
    llogos.write_random_model(folder, cfg, seed=seed)
    return pm.load_folder(folder)


def test_zeroed_output_projections_leave_the_embedding(tmp_path, llogos):
    import tiny_configs as tc
    cfg, w = _tiny(tmp_path, tc.TINY_A, llogos)
    for name in w:
        if name.endswith("o_proj.weight") or name.endswith("down_proj.weight"):
            w[name] = np.zeros_like(w[name])
    toks = [3, 9, 200, 17]
    want = pm.linear(pm.rms_norm(pm.embedding(w["model.embed_tokens.weight"], toks), w["model.norm.weight"], cfg.eps),
                     w["lm_head.weight"])
    assert np.allclose(pm.forward(cfg, w, toks), want)


def test_future_tokens_do_not_change_earlier_logits(tmp_path, llogos):
    import tiny_configs as tc
    cfg, w = _tiny(tmp_path, tc.TINY_B, llogos)
    a = pm.forward(cfg, w, [5, 6, 7, 8, 9, 10])
    b = pm.forward(cfg, w, [5, 6, 7, 8, 300, 11])
    assert np.allclose(a[:4], b[:4]) and not np.allclose(a[4], b[4])


def test_tied_head_is_the_embedding(tmp_path, llogos):
    import tiny_configs as tc
    cfg, w = _tiny(tmp_path, tc.TINY_B, llogos)
    assert cfg.tied and "lm_head.weight" not in w
    a = pm.forward(cfg, w, [1, 2, 3])
    w2 = dict(w); w2["lm_head.weight"] = w["model.embed_tokens.weight"].copy()
    cfg.tied = False
    assert np.allclose(a, pm.forward(cfg, w2, [1, 2, 3]))


def test_options_of_the_configurations_are_read(tmp_path, llogos):
    import tiny_configs as tc
    a, _ = _tiny(tmp_path / "a", tc.TINY_A, llogos)
    b, wb = _tiny(tmp_path / "b", tc.TINY_B, llogos)
    c, _ = _tiny(tmp_path / "c", tc.TINY_C, llogos)
    wcfg, _ = _tiny(tmp_path / "w", tc.TINY_W, llogos)
    assert a.bias and not a.qk_norm and a.head_dim == 16
    assert b.qk_norm and not b.bias and b.head_dim == 32 and "model.layers.0.self_attn.q_norm.weight" in wb
    assert c.rope_scaling["rope_type"] == "llama3" and not np.allclose(c.frequencies(), pm.rope_frequencies(48, 5e5))
    assert wcfg.windows == [0, 70, 70]


# ---- sampling (vectors of tests/Daisi.Llogos.Tests/Inference/SamplerTests.cs) ----
def test_sampler_vectors():
    assert pm.sample([1., 5., 3., 2.], 0.5, temperature=0, repetition_penalty=1.0) == 1          # :8-18
    big = np.zeros(1000); big[742] = 10
    assert pm.sample(big, 0.5, temperature=0, repetition_penalty=1.0) == 742                       # :20-31
    assert pm.argmax_first([3., 3., 3.]) == 0
    rng = np.random.default_rng(0)
    us = rng.random(1000)
    lo = [pm.sample([2., 1., .5, .1], u, temperature=0.1, top_k=0, top_p=1.0, repetition_penalty=1.0) for u in us]
    hi = [pm.sample([2., 1., .5, .1], u, temperature=2.0, top_k=0, top_p=1.0, repetition_penalty=1.0) for u in us]
    assert lo.count(0) > 900 and hi.count(0) < 600                                                 # :33-52
    tk = [pm.sample([5., 4., 3., 2., 1., 0., -1., -2.], u, temperature=1.0, top_k=3, top_p=1.0,
                    repetition_penalty=1.0) for u in us]
    assert set(tk) == {0, 1, 2}                                                                    # :54-70
    tp = [pm.sample([10., 1., 0., -1.], u, temperature=1.0, top_k=0, top_p=0.5, repetition_penalty=1.0) for u in us[:500]]
    assert tp.count(0) > 400                                                                       # :72-84
    assert pm.sample([3., 3., 3., 3.], 0.5, temperature=0, repetition_penalty=2.0, history=[0, 1]) >= 2   # :86-103


def test_sampler_draw_is_the_inverse_cdf_in_descending_order():
    logits = np.log(np.array([0.1, 0.6, 0.3]))
    kw = dict(temperature=1.0, top_k=0, top_p=1.0, repetition_penalty=1.0)
    assert pm.sample(logits, 0.59, **kw) == 1 and pm.sample(logits, 0.61, **kw) == 2 and pm.sample(logits, 0.95, **kw) == 0
    assert pm.sample(logits, 0.95, min_p=0.2, **kw) == 2                  # 0.1 < 0.2 * 0.6 is dropped
    kw["top_p"] = 0.7
    assert pm.sample(logits, 0.99, **kw) == 2                             # {0.6, 0.3} kept, renormalised
