"""The plain implementation is pinned by what fixes it beside the reference's text: vectors
the reference's tests hold, special cases that reduce to a library routine, and invariants.
Each check is chosen so that a plausible mistake fails it (named in its docstring)."""
import math

import numpy as np
import pytest

import plain_model as pm


# ---------------------------------------------------------------- RMSNorm
def test_rmsnorm_reference_vector():
    """Input and weight of crates/model-ops/src/ops/rmsnorm.rs:271-283 (linspace [-1,1] over
    4x64, w_c = 1 + 0.01c, eps 1e-5) against its CPU form :204-217 written out as loops."""
    n, h, eps = 4, 64, 1e-5
    x = np.array([2.0 * i / (n * h - 1) - 1.0 for i in range(n * h)]).reshape(n, h)
    w = np.array([1.0 + 0.01 * c for c in range(h)])
    want = np.zeros((n, h))
    for r in range(n):
        rms = math.sqrt(sum(v * v for v in x[r]) / h + eps)
        for c in range(h):
            want[r, c] = x[r, c] / rms * w[c]
    np.testing.assert_allclose(pm.rmsnorm(x, w, eps), want, rtol=1e-12, atol=1e-14)


def test_rmsnorm_eps_is_inside_the_root_and_added_to_the_mean():
    """x == c, w == 1 gives c / sqrt(c^2 + eps).  eps outside the root, or added to the sum
    instead of the mean, gives another number when eps is large."""
    c, eps, h = 0.5, 0.3, 16
    got = pm.rmsnorm(np.full((1, h), c), np.ones(h), eps)
    np.testing.assert_allclose(got, c / math.sqrt(c * c + eps), rtol=1e-14)
    assert abs(got[0, 0] - c / (math.sqrt(c * c) + eps)) > 1e-2
    assert abs(got[0, 0] - c / math.sqrt(c * c + eps / h)) > 1e-2


def test_rmsnorm_scale_invariance_and_unit_rms():
    rng = np.random.default_rng(0)
    x = rng.normal(size=(3, 40))
    y = pm.rmsnorm(x, np.ones(40), 0.0)
    np.testing.assert_allclose(np.sqrt((y * y).mean(-1)), 1.0, rtol=1e-12)
    np.testing.assert_allclose(pm.rmsnorm(7.0 * x, np.ones(40), 0.0), y, rtol=1e-12)


# ---------------------------------------------------------------- rotation
def test_rope_reference_vector_as_complex_multiplication():
    """Sizes of crates/model-ops/src/ops/rope.rs:204-233 (head 128, theta 1e6, positions
    [0, 7, 31, 128], x = cos(0.013 i - 0.7)), here with the whole head rotated: the two halves
    are the real and imaginary parts of numbers multiplied by e^{i phi}."""
    n, heads, hd, theta = 4, 2, 128, 1e6
    x = np.cos(0.013 * np.arange(n * heads * hd) - 0.7).reshape(n, heads, hd)
    pos = np.array([0, 7, 31, 128])
    got = pm.rope_neox(x, pos, theta)
    half = hd // 2
    z = x[..., :half] + 1j * x[..., half:]
    phi = pos[:, None] * theta ** (-2.0 * np.arange(half) / hd)
    zr = z * np.exp(1j * phi)[:, None, :]
    np.testing.assert_allclose(got[..., :half], zr.real, atol=1e-12)
    np.testing.assert_allclose(got[..., half:], zr.imag, atol=1e-12)


def test_rope_partial_reference_vector():
    """The reference's own case rotates 64 of 128 dims (rope.rs:204-233): the upper 64 pass
    through and the pairs are (i, i + 32)."""
    x = np.cos(0.013 * np.arange(4 * 2 * 128) - 0.7).reshape(4, 2, 128)
    got = pm.rope_neox(x, [0, 7, 31, 128], 1e6, rotated_dims=64)
    np.testing.assert_array_equal(got[..., 64:], x[..., 64:])
    np.testing.assert_array_equal(got[0], x[0])                       # position 0 is the identity
    i = 5
    phi = 7 * 1e6 ** (-2.0 * i / 64)
    want = x[1, 0, i] * math.cos(phi) - x[1, 0, i + 32] * math.sin(phi)
    assert abs(got[1, 0, i] - want) < 1e-12


def test_rope_pairs_split_half_not_interleaved():
    """A one-hot input at dim 1 moves weight to dim 1 + hd/2 (split halves).  Interleaved
    pairing (crates/kernels-hip/src/kernels/rope_f16.cu:20-47, the counter-example) would move
    it to dim 0."""
    hd = 16
    x = np.zeros((1, 1, hd))
    x[0, 0, 1] = 1.0
    y = pm.rope_neox(x, [3], 10000.0)
    nz = set(np.nonzero(np.abs(y[0, 0]) > 1e-12)[0])
    assert nz == {1, 1 + hd // 2}
    phi = 3 * 10000.0 ** (-2.0 / hd)
    np.testing.assert_allclose(y[0, 0, 1], math.cos(phi), atol=1e-12)
    np.testing.assert_allclose(y[0, 0, 1 + hd // 2], math.sin(phi), atol=1e-12)   # sign of sin


def test_rope_preserves_norms_and_depends_on_distance_only():
    rng = np.random.default_rng(1)
    q = rng.normal(size=(1, 1, 24))
    k = rng.normal(size=(1, 1, 24))
    np.testing.assert_allclose(np.linalg.norm(pm.rope_neox(q, [11], 1e4)), np.linalg.norm(q), rtol=1e-12)
    dots = [float((pm.rope_neox(q, [m], 1e4) * pm.rope_neox(k, [m - 5], 1e4)).sum()) for m in (5, 9, 100)]
    np.testing.assert_allclose(dots, dots[0], rtol=1e-10)
    other = float((pm.rope_neox(q, [9], 1e4) * pm.rope_neox(k, [3], 1e4)).sum())
    assert abs(other - dots[0]) > 1e-6


def test_rope_frequency_ladder_by_hand():
    """theta = 10^4 and 8 rotated dims give the frequencies 1, 1/10, 1/100, 1/1000 (theta^(-2i/rot):
    the exponent steps by 2/rot, starts at 0 and stops one step short of 1), so position 1000 turns
    pair 3 by exactly one radian and position 10 turns pair 1 by one radian.  An exponent i/rot, or
    2(i+1)/rot, or one taken over the head size instead of the rotated dims, fails."""
    hd, rot = 12, 8
    for pair, pos in ((0, 1), (1, 10), (2, 100), (3, 1000)):
        x = np.zeros((1, 1, hd))
        x[0, 0, pair] = 1.0
        y = pm.rope_neox(x, [pos], 1e4, rotated_dims=rot)[0, 0]
        np.testing.assert_allclose([y[pair], y[pair + rot // 2]], [math.cos(1.0), math.sin(1.0)], atol=1e-9)
    # measured from the function itself: the angle a pair turns by at position 1 is its frequency
    theta, rot = 5e5, 24
    freqs = []
    for pair in range(rot // 2):
        x = np.zeros((1, 1, rot))
        x[0, 0, pair] = 1.0
        y = pm.rope_neox(x, [1], theta)[0, 0]
        freqs.append(math.atan2(y[pair + rot // 2], y[pair]))
    assert freqs[0] == 1.0
    ratios = np.array(freqs[1:]) / np.array(freqs[:-1])
    np.testing.assert_allclose(ratios, ratios[0], rtol=1e-9)                      # a geometric ladder
    np.testing.assert_allclose(freqs[-1] * ratios[0], 1.0 / theta, rtol=1e-9)    # whose next rung would be 1 / theta


# ---------------------------------------------------------------- attention
def test_default_scale_is_the_library_routine_s():
    """Without rotation, window or grouping, attention with the default scale is torch's
    scaled_dot_product_attention with ITS default scale (1 / sqrt(head size)) and a causal mask."""
    import torch
    rng = np.random.default_rng(12)
    n, nh, hd = 11, 3, 20
    q, k, v = (rng.normal(size=(n, nh, hd)) for _ in range(3))
    got = pm.attention(q, k, v, np.arange(n), pm.default_scale(hd), 0)
    tq, tk, tv = (torch.from_numpy(a).permute(1, 0, 2)[None] for a in (q, k, v))     # [1, heads, n, hd]
    want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True)[0].permute(1, 0, 2).numpy()
    np.testing.assert_allclose(got, want, atol=1e-12)
    assert abs(pm.default_scale(64) - 0.125) < 1e-15


def _library_attention(q, k, v, scale, mask):
    """softmax(Q K^T scale + mask) V with heads already matched."""
    s = np.einsum("ihd,jhd->hij", q, k) * scale + mask[None]
    s = s - s.max(-1, keepdims=True)
    p = np.exp(s)
    p = p / p.sum(-1, keepdims=True)
    return np.einsum("hij,jhd->ihd", p, v)


def _causal_mask(n, window=0):
    i, j = np.arange(n)[:, None], np.arange(n)[None, :]
    ok = (j <= i) & ((j >= i - window + 1) if window > 0 else True)
    return np.where(ok, 0.0, -np.inf)


def test_attention_is_masked_softmax_for_plain_heads():
    rng = np.random.default_rng(2)
    n, nh, hd = 9, 3, 8
    q, k, v = (rng.normal(size=(n, nh, hd)) for _ in range(3))
    got = pm.attention(q, k, v, np.arange(n), 0.37, 0)
    np.testing.assert_allclose(got, _library_attention(q, k, v, 0.37, _causal_mask(n)), atol=1e-12)


def test_attention_grouped_heads_equal_repeated_keys():
    """Query heads g*k .. g*k+g-1 read key/value head k (kv_head = q_head // group):
    the same as repeating K and V over the group.  A modulo head map fails."""
    rng = np.random.default_rng(3)
    n, nh, nkv, hd = 7, 6, 2, 4
    q = rng.normal(size=(n, nh, hd))
    k, v = (rng.normal(size=(n, nkv, hd)) for _ in range(2))
    got = pm.attention(q, k, v, np.arange(n), 0.5, 0)
    kr, vr = np.repeat(k, nh // nkv, axis=1), np.repeat(v, nh // nkv, axis=1)
    np.testing.assert_allclose(got, _library_attention(q, kr, vr, 0.5, _causal_mask(n)), atol=1e-12)


def test_attention_window_counts_the_query_itself():
    """Window 4 at position 7 sees keys 4..7 (crates/ops/tests/swa_softcap_parity.rs:194-262,
    t_start = 7 - 4 + 1).  An off-by-one window (3 or 5 keys) fails."""
    rng = np.random.default_rng(4)
    n, hd = 8, 64
    q, k, v = (rng.uniform(-0.5, 0.5, size=(n, 1, hd)) for _ in range(3))
    got = pm.attention(q, k, v, np.arange(n), 1 / math.sqrt(hd), 4)[7, 0]
    s = (k[4:8, 0] @ q[7, 0]) / math.sqrt(hd)
    p = np.exp(s - s.max())
    np.testing.assert_allclose(got, (p / p.sum()) @ v[4:8, 0], atol=1e-12)
    np.testing.assert_allclose(pm.attention(q, k, v, np.arange(n), 1.0, 4),
                               _library_attention(q, k, v, 1.0, _causal_mask(n, 4)), atol=1e-12)


def test_attention_special_cases():
    rng = np.random.default_rng(5)
    n, nh, hd = 6, 2, 4
    q, k, v = (rng.normal(size=(n, nh, hd)) for _ in range(3))
    pos = np.arange(n)
    # one visible key: the output is that value row
    np.testing.assert_allclose(pm.attention(q, k, v, pos, 1.0, 1), v, atol=1e-12)
    np.testing.assert_allclose(pm.attention(q, k, v, pos, 1.0, 0)[0], v[0], atol=1e-12)
    # zero query: the mean of the visible values
    got = pm.attention(np.zeros_like(q), k, v, pos, 1.0, 0)
    np.testing.assert_allclose(got[3], v[:4].mean(0), atol=1e-12)
    # a window at least as long as the sequence changes nothing
    np.testing.assert_allclose(pm.attention(q, k, v, pos, 0.7, n), pm.attention(q, k, v, pos, 0.7, 0), atol=1e-12)
    # the scale multiplies the dot product
    a = pm.attention(q, k, v, pos, 0.5, 0)
    b = pm.attention(2 * q, k, v, pos, 0.25, 0)
    np.testing.assert_allclose(a, b, atol=1e-12)


def test_attention_in_batches_of_queries_is_the_whole_matrix():
    """More queries than one batch of the implementation's loop (256), with and without a window,
    against the library form over the whole score matrix; and queries at a few rows only."""
    rng = np.random.default_rng(6)
    n, nh, nkv, hd = 700, 4, 2, 8
    q = rng.normal(size=(n, nh, hd))
    k, v = (rng.normal(size=(n, nkv, hd)) for _ in range(2))
    kr, vr = np.repeat(k, 2, axis=1), np.repeat(v, 2, axis=1)
    pos = np.arange(n) + 11
    for window in (0, 1, 90, 300):
        want = _library_attention(q, kr, vr, 0.3, _causal_mask(n, window))
        np.testing.assert_allclose(pm.attention(q, k, v, pos, 0.3, window), want, atol=1e-12)
        rows = np.array([0, 255, 256, 511, 699, 3])
        got = pm.attention(q[rows], k, v, pos[rows], 0.3, window, key_positions=pos)
        np.testing.assert_allclose(got, want[rows], atol=1e-12)


# ---------------------------------------------------------------- feed-forward
def test_swiglu():
    """silu(g) = g * sigmoid(g); the gate, not the up projection, goes through it
    (crates/model-ops/src/ops/activation.rs:99-121)."""
    g = np.array([-30.0, -1.0, 0.0, 1.0, 30.0])
    np.testing.assert_allclose(pm.silu(g), g / (1 + np.exp(-g)), rtol=1e-14)
    assert pm.silu(0.0) == 0.0 and abs(pm.silu(30.0) - 30.0) < 1e-10 and abs(pm.silu(-30.0)) < 1e-10
    rng = np.random.default_rng(6)
    x = rng.normal(size=(3, 5))
    wg, wu, wd = rng.normal(size=(7, 5)), rng.normal(size=(7, 5)), rng.normal(size=(5, 7))
    gate, up = x @ wg.T, x @ wu.T
    np.testing.assert_allclose(pm.swiglu_mlp(x, wg, wu, wd), (gate * (1 / (1 + np.exp(-gate))) * up) @ wd.T, atol=1e-12)
    assert np.abs(pm.swiglu_mlp(x, wg, wu, wd) - (gate * pm.silu(up)) @ wd.T).max() > 1e-3


# ---------------------------------------------------------------- whole model
def _random_model(rng, L=2, H=16, nh=4, nkv=2, hd=6, I=20, V=30, window=None, tied=False):
    cfg = dict(hidden_size=H, num_hidden_layers=L, num_attention_heads=nh, num_key_value_heads=nkv,
               head_dim=hd, intermediate_size=I, vocab_size=V, rms_norm_eps=1e-5, rope_theta=1e4,
               sliding_window=window, tie_word_embeddings=tied)
    w = {"model.embed_tokens.weight": rng.normal(size=(V, H)), "model.norm.weight": 1 + 0.1 * rng.normal(size=H)}
    if not tied:
        w["lm_head.weight"] = rng.normal(size=(V, H))
    for l in range(L):
        p = f"model.layers.{l}."
        w[p + "input_layernorm.weight"] = 1 + 0.1 * rng.normal(size=H)
        w[p + "post_attention_layernorm.weight"] = 1 + 0.1 * rng.normal(size=H)
        w[p + "self_attn.q_proj.weight"] = rng.normal(size=(nh * hd, H)) * 0.3
        w[p + "self_attn.k_proj.weight"] = rng.normal(size=(nkv * hd, H)) * 0.3
        w[p + "self_attn.v_proj.weight"] = rng.normal(size=(nkv * hd, H)) * 0.3
        w[p + "self_attn.o_proj.weight"] = rng.normal(size=(H, nh * hd)) * 0.3
        w[p + "mlp.gate_proj.weight"] = rng.normal(size=(I, H)) * 0.3
        w[p + "mlp.up_proj.weight"] = rng.normal(size=(I, H)) * 0.3
        w[p + "mlp.down_proj.weight"] = rng.normal(size=(H, I)) * 0.3
    return cfg, w


def test_forward_with_silent_layers_is_head_of_normed_embedding():
    """Zero output and down projections: logits = Head(NormF(E[token])).  A norm in the wrong
    place (post-norm) or a missing final norm fails."""
    rng = np.random.default_rng(7)
    cfg, w = _random_model(rng)
    for l in range(2):
        w[f"model.layers.{l}.self_attn.o_proj.weight"][:] = 0
        w[f"model.layers.{l}.mlp.down_proj.weight"][:] = 0
    toks = [3, 9, 27, 1]
    e = w["model.embed_tokens.weight"][toks]
    want = pm.rmsnorm(e, w["model.norm.weight"], 1e-5) @ w["lm_head.weight"].T
    np.testing.assert_allclose(pm.forward(cfg, w, toks), want, atol=1e-12)


def test_forward_is_causal_and_shift_invariant():
    """Logits at a place do not depend on later tokens, and a shift of all positions changes
    nothing because only distances count.  Rotating V, or absolute-position leakage, fails."""
    rng = np.random.default_rng(8)
    cfg, w = _random_model(rng, window=5)
    toks = list(rng.integers(0, 30, 12))
    full = pm.forward(cfg, w, toks)
    np.testing.assert_allclose(pm.forward(cfg, w, toks[:7]), full[:7], atol=1e-10)
    np.testing.assert_allclose(pm.forward(cfg, w, toks, positions=np.arange(12) + 37), full, atol=1e-9)


def test_forward_layer_types_switch_the_window_per_layer():
    """``layer_types`` names the layers that have the window; all "sliding_attention" is the window
    everywhere, all "full_attention" is no window, and a mixture differs from both."""
    rng = np.random.default_rng(8)
    cfg, w = _random_model(rng, L=3, window=4)
    toks = list(rng.integers(0, 30, size=14))
    base = pm.forward(cfg, w, toks)
    np.testing.assert_array_equal(pm.forward(dict(cfg, layer_types=["sliding_attention"] * 3), w, toks), base)
    free = pm.forward(dict(cfg, sliding_window=None), w, toks)
    np.testing.assert_array_equal(pm.forward(dict(cfg, layer_types=["full_attention"] * 3), w, toks), free)
    mixed = pm.forward(dict(cfg, layer_types=["full_attention", "sliding_attention", "full_attention"]), w, toks)
    assert np.abs(mixed - base).max() > 1e-6 and np.abs(mixed - free).max() > 1e-6
    # only the second layer has the window: the same as a model whose other layers see everything
    np.testing.assert_array_equal(mixed[:4], free[:4])            # (no difference before the window bites)


def test_forward_at_some_rows_is_the_whole_forward_at_those_rows():
    rng = np.random.default_rng(10)
    for L, window in ((1, None), (3, 6), (2, None)):
        cfg, w = _random_model(rng, L=L, window=window)
        toks = list(rng.integers(0, 30, 40))
        full = pm.forward(cfg, w, toks)
        rows = [39, 0, 17, 18]
        np.testing.assert_allclose(pm.forward(cfg, w, toks, rows=rows), full[rows], atol=1e-11)
        np.testing.assert_allclose(pm.forward(cfg, w, toks, rows=rows, keep_layers=[]), pm.forward(cfg, w, toks, keep_layers=[])[rows], atol=1e-12)


def test_forward_tied_head_uses_the_embedding_table():
    rng = np.random.default_rng(9)
    cfg, w = _random_model(rng, tied=True)
    w2 = dict(w)
    cfg2 = dict(cfg, tie_word_embeddings=False)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"]
    toks = [1, 2, 3]
    np.testing.assert_allclose(pm.forward(cfg, w, toks), pm.forward(cfg2, w2, toks), atol=1e-14)


def test_forward_against_the_reference_snapshot():
    """crates/forward/tests/parity_snapshot_dense.rs:20-47: one layer, hidden 128, 4/2 heads of
    64, intermediate 256, vocabulary 64, deterministic weights
    (crates/forward/tests/common/mod.rs:80-86), unit norm gains, token 7 at position 0: the first
    16 logits and the argmax 56.  The reference stores its matrices in 8-bit blocks and its
    activations in 16-bit, so the match is loose (its own tolerance is 5e-3 against itself);
    a single token at position 0 pins neither rotation nor masks, but it does pin the layer
    order, the norms' places, the gate and the head map of V."""
    def det_signal(n, seed):
        i = np.arange(n, dtype=np.float32)
        s = np.float32(seed) * np.float32(0.013) + i * np.float32(0.027)
        return ((np.sin(s) + np.cos(s * np.float32(1.7))) * np.float32(0.1)).astype(np.float64)

    V, H, I, nh, nkv, hd = 64, 128, 256, 4, 2, 64
    cfg = dict(hidden_size=H, num_hidden_layers=1, num_attention_heads=nh, num_key_value_heads=nkv,
               head_dim=hd, intermediate_size=I, vocab_size=V, rms_norm_eps=1e-5, rope_theta=10000.0)
    p = "model.layers.0."
    w = {
        "model.embed_tokens.weight": det_signal(V * H, 1).reshape(V, H),
        "lm_head.weight": det_signal(V * H, 9).reshape(V, H),
        "model.norm.weight": np.ones(H),
        p + "input_layernorm.weight": np.ones(H),
        p + "post_attention_layernorm.weight": np.ones(H),
        p + "self_attn.q_proj.weight": det_signal(nh * hd * H, 101).reshape(nh * hd, H),
        p + "self_attn.k_proj.weight": det_signal(nkv * hd * H, 102).reshape(nkv * hd, H),
        p + "self_attn.v_proj.weight": det_signal(nkv * hd * H, 103).reshape(nkv * hd, H),
        p + "self_attn.o_proj.weight": det_signal(H * nh * hd, 104).reshape(H, nh * hd),
        p + "mlp.gate_proj.weight": det_signal(I * H, 105).reshape(I, H),
        p + "mlp.up_proj.weight": det_signal(I * H, 106).reshape(I, H),
        p + "mlp.down_proj.weight": det_signal(H * I, 107).reshape(H, I),
    }
    want = np.array([-0.27348816, -0.6983838, -0.4945717, -0.20793961, -0.41295117, 0.44879973,
                     -0.12378508, 0.9048374, 0.12987937, 0.9078851, 0.19723168, 0.42451006,
                     0.074222, -0.29097384, -0.09338939, -0.86321926])
    got = pm.forward(cfg, w, [7])[0]
    assert np.abs(got[:16] - want).max() < 2e-2, np.abs(got[:16] - want).max()
    # four logits (7, 9, 38, 56) lie within 0.008 of each other at the top, closer than the
    # reference's quantisation error, so its argmax 56 must be one of the near-maximal entries
    assert got[56] > got.max() - 2e-2
    assert np.corrcoef(got[:16], want)[0, 1] > 0.9995


# ---------------------------------------------------------------- sampling
def test_xoshiro_matches_hand_computed_values():
    """State (1, 2, 3, 4): the first output is rotl(2 * 5, 7) * 9 = 11520, and the state moves
    to (7, 0, 262146, 211106232532992)."""
    g = pm.Xoshiro(0)
    g.s = [1, 2, 3, 4]
    assert g.next_u64() == 11520
    assert g.s == [7, 0, 262146, 211106232532992]
    g2 = pm.Xoshiro(42)
    vals = [g2.next_f32() for _ in range(1000)]
    assert all(0.0 <= v < 1.0 for v in vals) and 0.4 < sum(vals) / 1000 < 0.6
    assert [pm.Xoshiro(42).next_u64() for _ in range(2)] == [pm.Xoshiro(42).next_u64()] * 2


def test_seeding_vector_for_seed_zero():
    """The four state words for seed 0, written out.  The first is SplitMix64's published first output
    from state 0 (0xE220A8397B1DCDAF: its increment added once, then its mixer).  The reference's
    loop (crates/runtime/src/sampling.rs:116-131) then differs from SplitMix64 proper: it does not add
    the increment again but mixes the running value in place (the value before the last xor-shift is
    carried on), so the second word is NOT SplitMix64's second output 0x6E789E6AA1B965F4.  The words are
    recomputed here with wrapping 64-bit machine arithmetic, step by step, not with masked big integers."""
    want = [0xE220A8397B1DCDAF, 0x622CF263EEB1289A, 0xC17A83783EC77EE4, 0xCCF1FA6DFE5D7959]
    assert pm.Xoshiro(0).s == want
    assert pm.Xoshiro(0).s[1] != 0x6E789E6AA1B965F4
    u = np.uint64
    with np.errstate(over="ignore"):
        x = u(0) + u(0x9E3779B97F4A7C15)
        words = []
        for _ in range(4):
            x = x ^ (x >> u(30))
            x = x * u(0xBF58476D1CE4E5B9)
            x = x ^ (x >> u(27))
            x = x * u(0x94D049BB133111EB)
            words.append(int(x ^ (x >> u(31))))
    assert words == want
    # and the first numbers drawn from that state: (1 + 2^-24 steps in [0, 1))
    g = pm.Xoshiro(0)
    first = g.next_u64()
    s1 = want[1]
    by_hand = (((s1 * 5) % 2 ** 64 << 7 | (s1 * 5) % 2 ** 64 >> 57) % 2 ** 64 * 9) % 2 ** 64
    assert first == by_hand
    assert pm.Xoshiro(0).next_f32() == (by_hand >> 40) / 2 ** 24


def test_sampler_rules():
    """The cases of crates/runtime/src/sampling.rs:752-939."""
    logits = np.array([0.1, 2.0, -1.0, 1.9, 0.5], dtype=np.float32)
    assert pm.sample(logits, pm.Xoshiro(1)) == 1                                   # greedy
    assert pm.sample(np.array([1.0, 3.0, 3.0], dtype=np.float32), pm.Xoshiro(1)) == 1   # first max
    a = [pm.sample(logits, pm.Xoshiro(7), temperature=0.8) for _ in range(3)]
    assert a[0] == a[1] == a[2]                                                    # same seed, same token
    g = pm.Xoshiro(3)
    draws = {pm.sample(logits, g, temperature=1.0, top_k=2) for _ in range(1000)}
    assert draws == {1, 3}
    g = pm.Xoshiro(4)
    draws = {pm.sample(logits, g, temperature=1.0, top_p=0.5) for _ in range(1000)}
    assert draws == {1, 3}        # p(1)=.41, p(3)=.37: the prefix reaches 0.5 with two
    g = pm.Xoshiro(5)
    draws = {pm.sample(logits, g, temperature=1.0, min_p=0.5) for _ in range(1000)}
    assert draws == {1, 3}        # p(4) / p(1) = 0.22 < 0.5
    # penalties flip the argmax
    assert pm.sample(logits, pm.Xoshiro(1), history=[1], repetition_penalty=2.0) == 3
    assert pm.sample(logits, pm.Xoshiro(1), history=[1], presence_penalty=0.5) == 3
    assert pm.sample(logits, pm.Xoshiro(1), history=[1, 1, 1], frequency_penalty=0.1) == 3
    assert pm.sample(logits, pm.Xoshiro(1), logit_bias={2: 10.0}) == 2
    # a negative logit is multiplied, not divided
    neg = pm.apply_penalties(np.array([-1.0, 1.0], dtype=np.float32), [0, 1], repetition_penalty=2.0)
    np.testing.assert_allclose(neg, [-2.0, 0.5])


def test_sampler_frequencies_follow_softmax():
    logits = np.array([0.0, 1.0, 2.0], dtype=np.float32)
    g = pm.Xoshiro(11)
    n = 6000
    counts = np.bincount([pm.sample(logits, g, temperature=0.7) for _ in range(n)], minlength=3) / n
    p = np.exp(logits / 0.7)
    p /= p.sum()
    assert np.abs(counts - p).max() < 0.03
