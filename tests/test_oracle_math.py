"""Pins the oracle's operators against what the mathematics fixes, independently of any fixture."""
import numpy as np

from metrics import rel_l2
from model_spec import normal_f32


def np_softmax(x):
    x = x.astype(np.float64)
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def test_linear_matches_numpy(oracle_mod):
    x = normal_f32((13, 70), 1, 1)
    W = normal_f32((29, 70), 1, 2)
    assert rel_l2(oracle_mod.linear(x, W), x.astype(np.float64) @ W.astype(np.float64).T) < 1e-6


def test_adaln_zero_modulation_is_layernorm(oracle_mod):
    x = normal_f32((9, 384), 1, 3, 2.0, 5.0)
    z = np.zeros(384, np.float32)
    y = oracle_mod.adaln(x, z, z)
    assert np.abs(y.mean(axis=1)).max() < 1e-5
    assert np.abs(y.var(axis=1) - 1.0).max() < 1e-4          # biased variance, eps 1e-6
    sh = normal_f32((384,), 1, 4)
    sc = normal_f32((384,), 1, 5)
    assert rel_l2(oracle_mod.adaln(x, sh, sc), (1.0 + sc) * y + sh) < 1e-6


def test_qk_norm_unit_rms(oracle_mod):
    q = normal_f32((6, 3 * 128), 1, 6, 0.0, 7.0)
    one = np.ones(128, np.float32)
    gq, gk = oracle_mod.qk_norm(q, q * 0.01, one, 2 * one, 3, 128)
    rms = np.sqrt((gq.reshape(6, 3, 128) ** 2).mean(-1))
    assert np.abs(rms - 1).max() < 1e-4
    rms_k = np.sqrt((gk.reshape(6, 3, 128) ** 2).mean(-1))
    assert np.abs(rms_k - 2).max() < 1e-2      # eps matters a little at small magnitude


def test_rope_is_pairwise_rotation(oracle_mod):
    c, s = oracle_mod.rope_image(5, 7, 32, 2000.0, 0)
    # duplicated on (2d, 2d+1), unit modulus, identity on the T and L axes of image tokens
    assert np.array_equal(c[:, 0::2], c[:, 1::2]) and np.array_equal(s[:, 0::2], s[:, 1::2])
    assert np.abs(c * c + s * s - 1).max() < 1e-6
    assert np.all(c[:, :32] == 1) and np.all(s[:, :32] == 0) and np.all(c[:, 96:] == 1)
    # closed form: angle = pos * theta^(-2d/32); rows -> axis 1, cols -> axis 2
    d = np.arange(16)
    f = 2000.0 ** (-2.0 * d / 32.0)
    tok = 3 * 7 + 4                                      # row 3, col 4
    np.testing.assert_allclose(c[tok, 32:64:2], np.cos(3 * f), atol=1e-5)
    np.testing.assert_allclose(s[tok, 64:96:2], np.sin(4 * f), atol=1e-5)
    ct, st = oracle_mod.rope_text(11)
    assert np.all(ct[:, :96] == 1) and np.all(st[:, :96] == 0)
    np.testing.assert_allclose(st[10, 96::2], np.sin(10 * f), atol=1e-5)
    cr, sr = oracle_mod.rope_image(2, 2, 32, 2000.0, 10)
    np.testing.assert_allclose(cr[3, 0:32:2], np.cos(10 * f), atol=1e-5)
    # application: complex multiplication per pair, norm preserving
    x = normal_f32((35, 2 * 128), 1, 7)
    y = oracle_mod.apply_rope(x, c, s, 2, 128)
    xc = x.reshape(35, 2, 64, 2)
    z = (xc[..., 0] + 1j * xc[..., 1]) * (c[:, None, 0::2] + 1j * s[:, None, 0::2])
    want = np.stack([z.real, z.imag], -1).reshape(35, 256)
    assert rel_l2(y, want) < 1e-6
    np.testing.assert_allclose(np.linalg.norm(y, axis=1), np.linalg.norm(x, axis=1), rtol=1e-5)


def test_attention_closed_forms(oracle_mod):
    heads, hd = 3, 128
    q = normal_f32((10, heads * hd), 1, 8)
    v1 = normal_f32((1, heads * hd), 1, 9)
    # one key: output is that value row regardless of scores
    out = oracle_mod.attention(q, v1 * 3, v1, heads, hd)
    assert rel_l2(out, np.repeat(v1, 10, 0)) < 1e-6
    # identical keys: uniform weights -> mean of V
    k = np.repeat(normal_f32((1, heads * hd), 1, 10), 17, 0)
    v = normal_f32((17, heads * hd), 1, 11)
    out = oracle_mod.attention(q, k, v, heads, hd)
    assert rel_l2(out, np.repeat(v.mean(0, keepdims=True), 10, 0)) < 1e-5
    # brute force in float64, seq_q != seq_k
    k = normal_f32((23, heads * hd), 1, 12)
    v = normal_f32((23, heads * hd), 1, 13)
    want = np.empty((10, heads * hd))
    for h in range(heads):
        sl = slice(h * hd, (h + 1) * hd)
        p = np_softmax(q[:, sl].astype(np.float64) @ k[:, sl].astype(np.float64).T / np.sqrt(hd))
        want[:, sl] = p @ v[:, sl]
    assert rel_l2(oracle_mod.attention(q, k, v, heads, hd), want) < 1e-6


def test_timestep_embedding_closed_form(oracle_mod):
    t = 437.5
    e = oracle_mod.timestep_embedding(t)
    i = np.arange(128)
    f = np.exp(-np.log(10000.0) * i / 128.0)
    np.testing.assert_allclose(e[:128], np.cos(t * f), atol=2e-4)    # cos half first
    np.testing.assert_allclose(e[128:], np.sin(t * f), atol=2e-4)


def test_official_schedule_closed_form(oracle_mod):
    s = oracle_mod.official_schedule(4, 4096)
    assert s[0] == 1.0 and s[-1] == 0.0 and np.all(np.diff(s) < 0)
    a1, b1, a2, b2 = 8.73809524e-05, 1.89833333, 0.00016927, 0.45666666
    m200, m10 = a2 * 4096 + b2, a1 * 4096 + b1
    a = (m200 - m10) / 190.0
    mu = a * 4 + (m200 - 200 * a)
    assert abs(mu - 2.2912) < 1e-3
    t = np.array([0.75, 0.5, 0.25])
    np.testing.assert_allclose(s[1:4], np.exp(mu) / (np.exp(mu) + (1 / t - 1)), rtol=1e-5)
    # beyond 4300 image tokens mu is the single line a2*n+b2
    s5 = oracle_mod.official_schedule(2, 5000)
    mu5 = a2 * 5000 + b2
    np.testing.assert_allclose(s5[1], np.exp(mu5) / (np.exp(mu5) + 1.0), rtol=1e-5)


def test_silu_softmax(oracle_mod):
    x = normal_f32((64,), 1, 14, 0.0, 4.0)
    np.testing.assert_allclose(oracle_mod.silu(x), x / (1 + np.exp(-x.astype(np.float64))), rtol=1e-5, atol=1e-6)
    m = normal_f32((4, 50), 1, 15, 0.0, 5.0)
    p = oracle_mod.softmax(m)
    np.testing.assert_allclose(p.sum(1), 1, atol=1e-5)
    np.testing.assert_allclose(p, np_softmax(m), atol=1e-6)


# ---- VAE operators ----

def test_conv2d_closed_forms(oracle_mod):
    x = normal_f32((3, 6, 5), 2, 1)
    # a kernel that is 1 at the centre of its own channel reproduces the input
    w = np.zeros((3, 3, 3, 3), np.float32)
    for c in range(3):
        w[c, c, 1, 1] = 1.0
    np.testing.assert_array_equal(oracle_mod.conv2d(x, w, None, 1), x)
    # a kernel that is 1 at (ky, kx) = (0, 2) reads the pixel one up and one to the right, zero outside
    w = np.zeros((1, 3, 3, 3), np.float32)
    w[0, 1, 0, 2] = 1.0
    want = np.zeros((6, 5), np.float32)
    want[1:, :-1] = x[1, :-1, 1:]
    np.testing.assert_array_equal(oracle_mod.conv2d(x, w, None, 1)[0], want)
    # all-ones 3x3 over a constant image counts the taps inside the image; bias adds on top
    ones = np.ones((1, 4, 4), np.float32)
    y = oracle_mod.conv2d(ones, np.ones((1, 1, 3, 3), np.float32), np.array([0.5], np.float32), 1)[0]
    assert y[0, 0] == 4.5 and y[0, 1] == 6.5 and y[1, 1] == 9.5 and y[3, 3] == 4.5
    # against a direct numpy evaluation
    w = normal_f32((4, 3, 3, 3), 2, 2)
    xp = np.pad(x.astype(np.float64), ((0, 0), (1, 1), (1, 1)))
    ref = np.zeros((4, 6, 5))
    for ky in range(3):
        for kx in range(3):
            ref += np.einsum("oc,chw->ohw", w[:, :, ky, kx].astype(np.float64), xp[:, ky:ky + 6, kx:kx + 5])
    assert rel_l2(oracle_mod.conv2d(x, w, None, 1), ref) < 1e-6


def test_downsample_and_patchify(oracle_mod):
    """The stride-2 step equals the plain 3x3 convolution of the image moved one pixel up and left
    (so that 'pad 1' supplies the zero row below / column on the right), sampled at the odd pixels;
    patchify and unpatchify are inverses, and patchify puts pixel (1, 0) of a 2x2 patch in channel 2."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal((3, 8, 10)).astype(np.float32)
    w = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)
    b = rng.standard_normal(4).astype(np.float32)
    down = oracle_mod.conv2d_down(x, w, b)
    assert down.shape == (4, 4, 5)
    full = oracle_mod.conv2d(x, w, b, 1)                 # full[y, x] reads rows y-1..y+1
    np.testing.assert_allclose(down, full[:, 1::2, 1::2], rtol=1e-5, atol=1e-5)
    # a kernel with a single 1 at (ky, kx) picks in[2y+ky, 2x+kx]
    for ky, kx in ((0, 0), (2, 1), (2, 2)):
        w1 = np.zeros((1, 1, 3, 3), np.float32)
        w1[0, 0, ky, kx] = 1.0
        xp = np.zeros((9, 11), np.float32)
        xp[:8, :10] = x[0]
        np.testing.assert_array_equal(oracle_mod.conv2d_down(x[:1], w1)[0], xp[ky::2, kx::2][:4, :5])
    p = oracle_mod.patchify(x)
    assert p.shape == (12, 4, 5)
    np.testing.assert_array_equal(oracle_mod.unpatchify(p), x)
    np.testing.assert_array_equal(p[2], x[0, 1::2, 0::2])
    np.testing.assert_array_equal(p[4 + 1], x[1, 0::2, 1::2])


def test_group_norm_statistics(oracle_mod):
    x = normal_f32((64, 6, 7), 2, 3, 1.5, 3.0)
    y = oracle_mod.group_norm(x, np.ones(64, np.float32), np.zeros(64, np.float32), 32, 1e-6)
    g = y.reshape(32, -1)
    assert np.abs(g.mean(axis=1)).max() < 1e-5 and np.abs(g.var(axis=1) - 1.0).max() < 1e-4
    gm, bt = normal_f32((64,), 2, 4), normal_f32((64,), 2, 5)
    assert rel_l2(oracle_mod.group_norm(x, gm, bt, 32, 1e-6), y * gm[:, None, None] + bt[:, None, None]) < 1e-6


# ---- Qwen3 text encoder ----

def test_qwen3_layer_matches_numpy(oracle_mod):
    """One layer of the tiny encoder against a float64 numpy evaluation of the same formulas."""
    from model_spec import QWEN3_TINY as cfg, make_qwen3_weights, bf16_to_f32
    W = make_qwen3_weights(cfg)
    o = oracle_mod.Qwen3Oracle(cfg, W)
    w = {k: bf16_to_f32(v).astype(np.float64) for k, v in W.items() if k.startswith("model.layers.1.")}
    g = lambda n: w["model.layers.1." + n]
    seq, H, hd, nh, nk = 7, cfg.hidden, cfg.head_dim, cfg.heads, cfg.kv_heads
    h = normal_f32((seq, H), 3, 1).astype(np.float64)
    mask = np.array([1, 1, 1, 1, 1, 0, 0])

    def rms(x, wt):
        return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + cfg.eps) * wt

    def rope(x, heads):
        x = x.reshape(seq, heads, hd).copy()
        i = np.arange(hd // 2)
        ang = np.arange(seq)[:, None] / cfg.rope_theta ** (2 * i / hd)[None, :]
        c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
        x0, x1 = x[..., :hd // 2].copy(), x[..., hd // 2:].copy()
        x[..., :hd // 2] = x0 * c - x1 * s
        x[..., hd // 2:] = x0 * s + x1 * c
        return x

    n = rms(h, g("input_layernorm.weight"))
    q = rope(rms((n @ g("self_attn.q_proj.weight").T).reshape(seq, nh, hd), g("self_attn.q_norm.weight")).reshape(seq, -1), nh)
    k = rope(rms((n @ g("self_attn.k_proj.weight").T).reshape(seq, nk, hd), g("self_attn.k_norm.weight")).reshape(seq, -1), nk)
    v = (n @ g("self_attn.v_proj.weight").T).reshape(seq, nk, hd)
    att = np.zeros((seq, nh, hd))
    for hh in range(nh):
        sc = q[:, hh] @ k[:, hh // (nh // nk)].T / np.sqrt(hd)
        sc[np.triu_indices(seq, 1)] = -1e9
        sc[:, mask == 0] = -1e9
        p = np.exp(sc - sc.max(axis=1, keepdims=True))
        att[:, hh] = (p / p.sum(axis=1, keepdims=True)) @ v[:, hh // (nh // nk)]
    h1 = h + att.reshape(seq, -1) @ g("self_attn.o_proj.weight").T
    n2 = rms(h1, g("post_attention_layernorm.weight"))
    gate, up = n2 @ g("mlp.gate_proj.weight").T, n2 @ g("mlp.up_proj.weight").T
    want = h1 + (gate / (1 + np.exp(-gate)) * up) @ g("mlp.down_proj.weight").T
    assert rel_l2(o.layer(1, h.astype(np.float32), mask), want) < 2e-6
    o.close()


def test_qwen3_causality_and_padding(oracle_mod):
    from model_spec import QWEN3_TINY as cfg, make_qwen3_weights
    o = oracle_mod.Qwen3Oracle(cfg, make_qwen3_weights(cfg))
    ids = np.array([3, 7, 299, 12, 5, 0, 0], np.int32)
    mask = np.array([1, 1, 1, 1, 1, 0, 0], np.int32)
    y = o.forward(ids, mask)
    assert y.shape == (7, 3 * cfg.hidden)
    ids2 = ids.copy()
    ids2[3] = 100                                        # a later token cannot change earlier positions
    y2 = o.forward(ids2, mask)
    np.testing.assert_array_equal(y[:3], y2[:3])
    assert np.abs(y[3:] - y2[3:]).max() > 1e-3
    ids3 = ids.copy()
    ids3[5:] = (44, 45)                                  # what sits in masked positions cannot change real positions
    np.testing.assert_array_equal(o.forward(ids3, mask)[:5], y[:5])
    # an id outside the vocabulary embeds as zeros (flux_qwen3.c:1053-1056): position 0 then stays zero in every captured layer
    y4 = o.forward(np.array([cfg.vocab, 4], np.int32), None)
    assert not y4[0].any() and np.abs(y4[1]).max() > 0
    o.close()
