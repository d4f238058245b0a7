#!/usr/bin/env python3
"""Regenerates tests/golden/*.npz by executing the reference's own C code.

Runs only in a container that has the reference checkout: `make -C oracle ref`
compiles the reference sources in place into oracle/_ref/libfluxref.so and this
script drives that library through ctypes on seeded synthetic inputs. The
fixtures hold inputs' seeds (in this script) and the reference's outputs (in
the .npz files); nothing of the reference's source text is stored.

    python tests/golden/make_golden.py            # everything except the 4B cases
    python tests/golden/make_golden.py --full     # also the two full-size c1 forwards (minutes, ~25 GB RAM)
"""
import argparse
import ctypes
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "flux2.c_amd"))
from model_spec import (TINY, KLEIN_4B, QWEN3_4B, make_weights, make_vae_weights, vae_test_image, make_qwen3_weights,  # noqa: E402
                        write_safetensors, normal_f32, bf16_to_f32)

c_f, c_i, vp = ctypes.c_float, ctypes.c_int, ctypes.c_void_p


class Cfg(ctypes.Structure):
    _fields_ = [(n, c_i) for n in ("hidden", "heads", "head_dim", "mlp", "n_double", "n_single",
                                   "text_dim", "channels", "axis_dim", "sincos_dim")] + [("rope_theta", c_f)]


class Ref(ctypes.Structure):
    _fields_ = [("latent", vp), ("h", c_i), ("w", c_i), ("t_offset", c_i)]


def load():
    L = ctypes.CDLL(os.path.join(ROOT, "oracle", "_ref", "libfluxref.so"))
    L.ref_model_new.restype = vp
    L.ref_model_new.argtypes = [ctypes.POINTER(Cfg)]
    L.ref_model_set_bf16.argtypes = [vp, ctypes.c_char_p, vp, ctypes.c_int64]
    L.ref_model_free.argtypes = [vp]
    L.ref_free.argtypes = [vp]
    for name in ("flux_transformer_forward", "flux_transformer_forward_with_refs",
                 "flux_transformer_forward_with_multi_refs", "flux_sample_euler",
                 "flux_sample_euler_with_refs", "flux_sample_euler_with_multi_refs",
                 "flux_sample_euler_cfg", "flux_sample_euler_cfg_with_refs",
                 "flux_sample_euler_cfg_with_multi_refs", "flux_linear_schedule",
                 "flux_power_schedule", "flux_official_schedule", "flux_init_noise",
                 "flux_sigmoid_schedule", "flux_resolution_schedule", "flux_sample_heun",
                 "flux_sample_euler_ancestral"):
        getattr(L, name).restype = vp
    L.flux_transformer_forward.argtypes = [vp, vp, c_i, c_i, vp, c_i, c_f]
    L.flux_transformer_forward_with_refs.argtypes = [vp, vp, c_i, c_i, vp, c_i, c_i, c_i, vp, c_i, c_f]
    L.flux_transformer_forward_with_multi_refs.argtypes = [vp, vp, c_i, c_i, vp, c_i, vp, c_i, c_f]
    L.flux_sample_euler.argtypes = [vp, vp, vp, c_i, c_i, c_i, c_i, vp, c_i, vp, c_i, vp]
    L.flux_sample_euler_with_refs.argtypes = [vp, vp, vp, c_i, c_i, c_i, c_i, vp, c_i, c_i, c_i, vp, c_i, vp, c_i, vp]
    L.flux_sample_euler_with_multi_refs.argtypes = [vp, vp, vp, c_i, c_i, c_i, c_i, vp, c_i, vp, c_i, vp, c_i, vp]
    L.flux_sample_euler_cfg.argtypes = [vp, vp, vp, c_i, c_i, c_i, c_i, vp, c_i, vp, c_i, c_f, vp, c_i, vp]
    L.flux_sample_euler_cfg_with_refs.argtypes = [vp, vp, vp, c_i, c_i, c_i, c_i, vp, c_i, c_i, c_i,
                                                  vp, c_i, vp, c_i, c_f, vp, c_i, vp]
    L.flux_sample_euler_cfg_with_multi_refs.argtypes = [vp, vp, vp, c_i, c_i, c_i, c_i, vp, c_i,
                                                        vp, c_i, vp, c_i, c_f, vp, c_i, vp]
    L.flux_sample_heun.argtypes = [vp, vp, c_i, c_i, c_i, c_i, vp, c_i, vp, c_i, vp]
    L.flux_sample_euler_ancestral.argtypes = [vp, vp, c_i, c_i, c_i, c_i, vp, c_i, vp, c_i, c_f, vp]
    L.flux_sigmoid_schedule.argtypes = [c_i, c_f]
    L.flux_resolution_schedule.argtypes = [c_i, c_i, c_i]
    L.flux_linear_schedule.argtypes = [c_i]
    L.flux_power_schedule.argtypes = [c_i, c_f]
    L.flux_official_schedule.argtypes = [c_i, c_i]
    L.flux_init_noise.argtypes = [c_i, c_i, c_i, c_i, ctypes.c_int64]
    L.flux_rng_seed.argtypes = [ctypes.c_uint64]
    L.flux_randn.argtypes = [vp, c_i]
    L.flux_linear_nobias.argtypes = [vp, vp, vp, c_i, c_i, c_i]
    L.flux_softmax.argtypes = [vp, c_i, c_i]
    L.flux_silu.argtypes = [vp, c_i]
    L.flux_flash_attention.argtypes = [vp, vp, vp, vp, c_i, c_i, c_i, c_i, c_f]
    L.flux_attention.argtypes = [vp, vp, vp, vp, c_i, c_i, c_i, c_i, c_i, c_f]
    L.ref_timestep_embedding.argtypes = [vp, c_f, c_i, c_f]
    L.ref_time_mlp.argtypes = [vp, vp, vp, vp, c_i, c_i]
    L.ref_rope_image.argtypes = [vp, vp, c_i, c_i, c_i, c_f, c_i]
    L.ref_rope_text.argtypes = [vp, vp, c_i, c_i, c_f]
    L.ref_apply_rope.argtypes = [vp, vp, vp, c_i, c_i, c_i]
    L.ref_adaln.argtypes = [vp, vp, vp, vp, c_i, c_i, c_f]
    L.ref_qk_norm.argtypes = [vp, vp, vp, vp, c_i, c_i, c_i, c_f]
    L.ref_gated_add.argtypes = [vp, vp, vp, c_i, c_i]
    L.ref_joint_attention.argtypes = [vp] + [vp] * 8 + [c_i, c_i]
    L.ref_mha.argtypes = [vp, vp, vp, vp, vp, c_i]
    L.ref_double_block.argtypes = [vp, c_i] + [vp] * 8 + [c_i, c_i]
    L.ref_single_block.argtypes = [vp, c_i] + [vp] * 6 + [c_i, c_i]
    return L


L = None


def P(a):
    return a.ctypes.data


def take(ptr, shape):
    n = int(np.prod(shape))
    out = np.ctypeslib.as_array(ctypes.cast(ptr, ctypes.POINTER(c_f)), shape=(n,)).copy().reshape(shape)
    L.ref_free(ptr)
    return out


def new_model(cfg, weights):
    c = Cfg(cfg.hidden, cfg.heads, cfg.head_dim, cfg.mlp, cfg.n_double, cfg.n_single, cfg.text_dim,
            cfg.channels, cfg.axis_dim, cfg.sincos_dim, cfg.rope_theta)
    m = L.ref_model_new(ctypes.byref(c))
    for name, a in weights.items():
        rc = L.ref_model_set_bf16(m, name.encode(), P(a), a.size)
        assert rc == 0, (name, rc)
    return m


def refs_array(refs):
    arr = (Ref * len(refs))()
    for i, (lat, h, w, t) in enumerate(refs):
        arr[i] = Ref(P(lat), h, w, t)
    return arr


# Seeds / shapes shared with tests/test_oracle_golden.py -------------------------------------------
SEED = 7
ANCESTRAL_SEED = 99     # flux_rng_seed() value set right before the ancestral sampler runs
ANCESTRAL_ETA = 0.7


def case_inputs(cfg):
    """Inputs of the TINY whole-model cases (regenerated identically by the tests)."""
    d = {}
    d["lat"] = normal_f32((cfg.channels, 4, 4), SEED, 100)
    d["txt"] = normal_f32((16, cfg.text_dim), SEED, 101)
    d["txt_u"] = normal_f32((12, cfg.text_dim), SEED, 102)
    d["ref1"] = normal_f32((cfg.channels, 2, 3), SEED, 103)
    d["ref2"] = normal_f32((cfg.channels, 3, 2), SEED, 104)
    return d


def ops_golden():
    g = {}
    # timestep embedding (t is pre-multiplied by 1000 by the caller)
    for t in (0.0, 250.0, 967.384, 1000.0):
        o = np.empty(256, np.float32)
        L.ref_timestep_embedding(P(o), t, 256, 10000.0)
        g[f"temb_{t}"] = o
    # rope tables
    for (ph, pw, toff) in ((4, 3, 0), (3, 5, 10), (2, 2, 20)):
        c = np.empty((ph * pw, 128), np.float32); s = np.empty_like(c)
        L.ref_rope_image(P(c), P(s), ph, pw, 32, 2000.0, toff)
        g[f"rope_img_{ph}_{pw}_{toff}_cos"] = c; g[f"rope_img_{ph}_{pw}_{toff}_sin"] = s
    c = np.empty((9, 128), np.float32); s = np.empty_like(c)
    L.ref_rope_text(P(c), P(s), 9, 32, 2000.0)
    g["rope_txt_9_cos"] = c; g["rope_txt_9_sin"] = s
    # apply rope: 5 tokens of a 4x3 grid table, 3 heads
    x = normal_f32((12, 3 * 128), SEED, 1)
    c = g["rope_img_4_3_0_cos"]; s = g["rope_img_4_3_0_sin"]
    y = x.copy(); L.ref_apply_rope(P(y), P(c), P(s), 12, 3, 128)
    g["apply_rope"] = y
    # adaln
    x = normal_f32((6, 256), SEED, 2, 0.3, 2.0); sh = normal_f32((256,), SEED, 3); sc = normal_f32((256,), SEED, 4)
    o = np.empty_like(x); L.ref_adaln(P(o), P(x), P(sh), P(sc), 6, 256, 1e-6)
    g["adaln"] = o
    # qk norm
    q = normal_f32((5, 256), SEED, 5); k = normal_f32((5, 256), SEED, 6, 0.0, 3.0)
    qw = normal_f32((128,), SEED, 7); kw = normal_f32((128,), SEED, 8)
    L.ref_qk_norm(P(q), P(k), P(qw), P(kw), 5, 2, 128, 1e-6)
    g["qknorm_q"] = q; g["qknorm_k"] = k
    # gated add
    o = normal_f32((4, 256), SEED, 9); gt = normal_f32((256,), SEED, 10); pr = normal_f32((4, 256), SEED, 11)
    L.ref_gated_add(P(o), P(gt), P(pr), 4, 256)
    g["gated_add"] = o
    # linear / softmax / silu
    x = normal_f32((7, 96), SEED, 12); W = normal_f32((40, 96), SEED, 13)
    y = np.empty((7, 40), np.float32); L.flux_linear_nobias(P(y), P(x), P(W), 7, 96, 40)
    g["linear"] = y
    x = normal_f32((5, 33), SEED, 14, 0.0, 4.0); L.flux_softmax(P(x), 5, 33); g["softmax"] = x
    x = normal_f32((300,), SEED, 15, 0.0, 3.0); L.flux_silu(P(x), 300); g["silu"] = x
    # attention: small (non-tiled flash path) and large (tiled path), seq_q != seq_k
    for tag, sq, sk in (("small", 12, 19), ("tiled", 70, 141)):
        q = normal_f32((sq, 256), SEED, 20); k = normal_f32((sk, 256), SEED, 21); v = normal_f32((sk, 256), SEED, 22)
        o = np.empty_like(q)
        L.flux_flash_attention(P(o), P(q), P(k), P(v), sq, sk, 2, 128, 1.0 / np.sqrt(128.0))
        g[f"flash_{tag}"] = o
    # naive attention in [heads, seq, hd] layout (third implementation)
    q = normal_f32((2, 12, 128), SEED, 23); k = normal_f32((2, 19, 128), SEED, 24); v = normal_f32((2, 19, 128), SEED, 25)
    o = np.empty_like(q)
    L.flux_attention(P(o), P(q), P(k), P(v), 1, 2, 12, 19, 128, 1.0 / np.sqrt(128.0))
    g["naive_attn"] = o
    # schedules
    for n in (1, 4, 7):
        g[f"sched_linear_{n}"] = take(L.flux_linear_schedule(n), (n + 1,))
    g["sched_power_5_2"] = take(L.flux_power_schedule(5, 2.0), (6,))
    for n, sl in ((4, 256), (4, 1024), (4, 4096), (50, 1024), (4, 5000), (1, 16), (28, 4300)):
        g[f"sched_official_{n}_{sl}"] = take(L.flux_official_schedule(n, sl), (n + 1,))
    for n, sh in ((4, 0.0), (7, 1.5), (1, -2.0)):
        g[f"sched_sigmoid_{n}_{sh}"] = take(L.flux_sigmoid_schedule(n, sh), (n + 1,))
    for n, hh, ww in ((4, 256, 256), (6, 512, 512), (5, 1024, 1024), (3, 2048, 256), (4, 768, 1024)):
        g[f"sched_resolution_{n}_{hh}_{ww}"] = take(L.flux_resolution_schedule(n, hh, ww), (n + 1,))
    # rng + noise
    L.flux_rng_seed(42); o = np.empty(64, np.float32); L.flux_randn(P(o), 64); g["randn_42"] = o
    g["noise_42_4x4"] = take(L.flux_init_noise(1, 128, 4, 4, 42), (128, 4, 4))
    g["noise_123_3x5"] = take(L.flux_init_noise(1, 128, 3, 5, 123), (128, 3, 5))
    return g


def model_golden(cfg, qk):
    g = {}
    W = make_weights(cfg, 42, 0.02, qk)
    m = new_model(cfg, W)
    H = cfg.hidden
    d = case_inputs(cfg)
    lat, txt, txt_u, ref1, ref2 = d["lat"], d["txt"], d["txt_u"], d["ref1"], d["ref2"]

    # time MLP
    e = np.empty(256, np.float32); L.ref_timestep_embedding(P(e), 500.0, 256, 10000.0)
    fc1 = bf16_to_f32(W["time_guidance_embed.timestep_embedder.linear_1.weight"])
    fc2 = bf16_to_f32(W["time_guidance_embed.timestep_embedder.linear_2.weight"])
    o = np.empty(H, np.float32); L.ref_time_mlp(P(o), P(e), P(fc1), P(fc2), 256, H); g["time_mlp"] = o

    # joint attention / mha through the model's work buffers
    iq = normal_f32((12, H), SEED, 30); ik = normal_f32((12, H), SEED, 31); iv = normal_f32((12, H), SEED, 32)
    tq = normal_f32((7, H), SEED, 33); tk = normal_f32((7, H), SEED, 34); tv = normal_f32((7, H), SEED, 35)
    io = np.empty_like(iq); to = np.empty_like(tq)
    assert L.ref_joint_attention(m, P(io), P(to), P(iq), P(ik), P(iv), P(tq), P(tk), P(tv), 12, 7) == 0
    g["joint_img"] = io; g["joint_txt"] = to
    o = np.empty_like(iq); assert L.ref_mha(m, P(o), P(iq), P(ik), P(iv), 12) == 0; g["mha"] = o

    # blocks with O(1) activations and modulation
    ic = np.empty((12, 128), np.float32); isn = np.empty_like(ic); L.ref_rope_image(P(ic), P(isn), 3, 4, 32, 2000.0, 0)
    tc = np.empty((7, 128), np.float32); ts = np.empty_like(tc); L.ref_rope_text(P(tc), P(ts), 7, 32, 2000.0)
    ih = normal_f32((12, H), SEED, 40); th = normal_f32((7, H), SEED, 41)
    im = normal_f32((6 * H,), SEED, 42, 0.0, 0.5); tm = normal_f32((6 * H,), SEED, 43, 0.0, 0.5)
    assert L.ref_double_block(m, 1, P(ih), P(th), P(im), P(tm), P(ic), P(isn), P(tc), P(ts), 12, 7) == 0
    g["dbl_img"] = ih; g["dbl_txt"] = th
    x = normal_f32((19, H), SEED, 44); temb = normal_f32((H,), SEED, 45, 0.0, 3.0)
    assert L.ref_single_block(m, 2, P(x), P(temb), P(ic), P(isn), P(tc), P(ts), 19, 7) == 0
    g["sgl"] = x

    # whole forwards
    n = cfg.channels * 16
    g["fwd_t1.0"] = take(L.flux_transformer_forward(m, P(lat), 4, 4, P(txt), 16, 1.0), (cfg.channels, 4, 4))
    g["fwd_t0.37"] = take(L.flux_transformer_forward(m, P(lat), 4, 4, P(txt), 16, 0.37), (cfg.channels, 4, 4))
    g["fwd_ref1"] = take(L.flux_transformer_forward_with_refs(m, P(lat), 4, 4, P(ref1), 2, 3, 10, P(txt), 16, 0.6),
                         (cfg.channels, 4, 4))
    ra = refs_array([(ref1, 2, 3, 10), (ref2, 3, 2, 20)])
    g["fwd_ref2"] = take(L.flux_transformer_forward_with_multi_refs(m, P(lat), 4, 4, ra, 2, P(txt), 16, 0.6),
                         (cfg.channels, 4, 4))

    # samplers
    s3 = take(L.flux_official_schedule(3, 16), (4,))
    z = lat.copy()
    g["euler3"] = take(L.flux_sample_euler(m, None, P(z), 1, cfg.channels, 4, 4, P(txt), 16, P(s3), 3, None),
                       (cfg.channels, 4, 4))
    g["euler3_ref1"] = take(L.flux_sample_euler_with_refs(m, None, P(z), 1, cfg.channels, 4, 4, P(ref1), 2, 3, 10,
                                                          P(txt), 16, P(s3), 3, None), (cfg.channels, 4, 4))
    g["euler3_ref2"] = take(L.flux_sample_euler_with_multi_refs(m, None, P(z), 1, cfg.channels, 4, 4, ra, 2,
                                                                P(txt), 16, P(s3), 3, None), (cfg.channels, 4, 4))
    g["cfg2"] = take(L.flux_sample_euler_cfg(m, None, P(z), 1, cfg.channels, 4, 4, P(txt), 16, P(txt_u), 12,
                                             4.0, P(s3), 2, None), (cfg.channels, 4, 4))
    g["cfg2_ref1"] = take(L.flux_sample_euler_cfg_with_refs(m, None, P(z), 1, cfg.channels, 4, 4, P(ref1), 2, 3, 10,
                                                            P(txt), 16, P(txt_u), 12, 4.0, P(s3), 2, None),
                          (cfg.channels, 4, 4))
    g["cfg2_ref2"] = take(L.flux_sample_euler_cfg_with_multi_refs(m, None, P(z), 1, cfg.channels, 4, 4, ra, 2,
                                                                  P(txt), 16, P(txt_u), 12, 4.0, P(s3), 2, None),
                          (cfg.channels, 4, 4))
    # second-order and stochastic samplers (no reference-image variants exist for these)
    g["heun3"] = take(L.flux_sample_heun(m, P(z), 1, cfg.channels, 4, 4, P(txt), 16, P(s3), 3, None),
                      (cfg.channels, 4, 4))
    g["heun1"] = take(L.flux_sample_heun(m, P(z), 1, cfg.channels, 4, 4, P(txt), 16, P(s3), 1, None),
                      (cfg.channels, 4, 4))
    L.flux_rng_seed(ANCESTRAL_SEED)
    g["ancestral3"] = take(L.flux_sample_euler_ancestral(m, P(z), 1, cfg.channels, 4, 4, P(txt), 16, P(s3), 3,
                                                         ANCESTRAL_ETA, None), (cfg.channels, 4, 4))
    g["ancestral3_eta0"] = take(L.flux_sample_euler_ancestral(m, P(z), 1, cfg.channels, 4, 4, P(txt), 16, P(s3), 3,
                                                              0.0, None), (cfg.channels, 4, 4))
    L.ref_model_free(m)
    return g


class FluxImage(ctypes.Structure):           # flux.h:73-78
    _fields_ = [("width", c_i), ("height", c_i), ("channels", c_i), ("data", ctypes.POINTER(ctypes.c_uint8))]


# shapes shared with tests/test_oracle_golden.py
VAE_OP_SEED = 21
VAE_DECODE_CASES = ((2, 2, 301), (3, 2, 302))     # latent h, w, seed
VAE_ENCODE_CASES = ((32, 32, 311), (48, 32, 312))   # image H, W, seed


def vae_golden():
    """The reference's convolution, group norm, upsample, patchify and unpatchify (flux_kernels.c) on
    small seeded tensors, and its VAE decoder and encoder (flux_vae_decode, flux_vae.c:690;
    flux_vae_encode, flux_vae.c:320) on the synthetic full-size VAE of model_spec.make_vae_weights."""
    import tempfile
    g = {}
    for fn in ("flux_conv2d", "flux_group_norm", "flux_upsample_nearest", "flux_unpatchify"):
        getattr(L, fn).restype = None
    L.flux_conv2d.argtypes = [vp, vp, vp, vp] + [c_i] * 9
    L.flux_group_norm.argtypes = [vp, vp, vp, vp, c_i, c_i, c_i, c_i, c_i, c_f]
    L.flux_upsample_nearest.argtypes = [vp, vp] + [c_i] * 6
    L.flux_unpatchify.argtypes = [vp, vp] + [c_i] * 5
    x = normal_f32((5, 7, 6), VAE_OP_SEED, 1)
    w3 = normal_f32((4, 5, 3, 3), VAE_OP_SEED, 2, 0.0, 0.2)
    w1 = normal_f32((4, 5, 1, 1), VAE_OP_SEED, 3, 0.0, 0.4)
    b = normal_f32((4,), VAE_OP_SEED, 4)
    o = np.empty((4, 7, 6), np.float32)
    L.flux_conv2d(P(o), P(x), P(w3), P(b), 1, 5, 4, 7, 6, 3, 3, 1, 1)
    g["conv3x3"] = o.copy()
    L.flux_conv2d(P(o), P(x), P(w1), P(b), 1, 5, 4, 7, 6, 1, 1, 1, 0)
    g["conv1x1"] = o.copy()
    L.flux_conv2d(P(o), P(x), P(w3), None, 1, 5, 4, 7, 6, 3, 3, 1, 1)
    g["conv3x3_nobias"] = o.copy()
    xg = normal_f32((64, 5, 3), VAE_OP_SEED, 5, 0.3, 2.0)
    gm, bt = normal_f32((64,), VAE_OP_SEED, 6, 1.0, 0.2), normal_f32((64,), VAE_OP_SEED, 7)
    og = np.empty_like(xg)
    L.flux_group_norm(P(og), P(xg), P(gm), P(bt), 1, 64, 5, 3, 32, 1e-4)
    g["group_norm"] = og
    xu = normal_f32((3, 4, 5), VAE_OP_SEED, 8)
    ou = np.empty((3, 8, 10), np.float32)
    L.flux_upsample_nearest(P(ou), P(xu), 1, 3, 4, 5, 2, 2)
    g["upsample"] = ou
    xp = normal_f32((12, 3, 2), VAE_OP_SEED, 9)
    op = np.empty((3, 6, 4), np.float32)
    L.flux_unpatchify(P(op), P(xp), 1, 3, 3, 2, 2)
    g["unpatchify"] = op
    L.flux_patchify.restype = None
    L.flux_patchify.argtypes = [vp, vp] + [c_i] * 5
    xq = normal_f32((3, 6, 4), VAE_OP_SEED, 10)
    oq = np.empty((12, 3, 2), np.float32)
    L.flux_patchify(P(oq), P(xq), 1, 3, 6, 4, 2)
    g["patchify"] = oq
    # the encoder's downsampling step (flux_vae.c:363-377): zeros below and on the right, then stride 2 without padding
    for tag, (H, W) in (("even", (8, 6)), ("odd", (7, 9))):
        xd = normal_f32((5, H, W), VAE_OP_SEED, 11)
        xpad = np.zeros((5, H + 1, W + 1), np.float32)
        xpad[:, :H, :W] = xd
        od = np.empty((4, (H - 2) // 2 + 1, (W - 2) // 2 + 1), np.float32)
        L.flux_conv2d(P(od), P(xpad), P(w3), P(b), 1, 5, 4, H + 1, W + 1, 3, 3, 2, 0)
        g[f"conv_down_{tag}"] = od

    L.safetensors_open.restype = vp
    L.safetensors_open.argtypes = [ctypes.c_char_p]
    L.safetensors_close.argtypes = [vp]
    L.flux_vae_load_safetensors.restype = vp
    L.flux_vae_load_safetensors.argtypes = [vp]
    L.flux_vae_decode.restype = vp
    L.flux_vae_decode.argtypes = [vp, vp, c_i, c_i, c_i]
    L.flux_vae_free.argtypes = [vp]
    L.flux_image_free.argtypes = [vp]
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "vae.safetensors")
        write_safetensors(path, make_vae_weights())
        sf = L.safetensors_open(path.encode())
        vae = L.flux_vae_load_safetensors(sf)
        L.safetensors_close(sf)
        assert vae
        for h, w, seed in VAE_DECODE_CASES:
            lat = normal_f32((128, h, w), seed, 1)
            ip = L.flux_vae_decode(vae, P(lat), 1, h, w)
            assert ip
            im = ctypes.cast(ip, ctypes.POINTER(FluxImage)).contents
            g[f"decode_{h}x{w}"] = np.ctypeslib.as_array(im.data, shape=(im.height, im.width, im.channels)).copy()
            L.flux_image_free(ip)
            print("vae decode", h, w, "std", g[f"decode_{h}x{w}"].std(), flush=True)
        L.flux_vae_encode.restype = ctypes.POINTER(ctypes.c_float)
        L.flux_vae_encode.argtypes = [vp, vp, c_i, c_i, c_i, ctypes.POINTER(c_i), ctypes.POINTER(c_i)]
        libc = ctypes.CDLL(None)
        libc.free.argtypes = [vp]
        for H, W, seed in VAE_ENCODE_CASES:
            img = vae_test_image(H, W, seed)
            oh, ow = c_i(0), c_i(0)
            lp = L.flux_vae_encode(vae, P(img), 1, H, W, ctypes.byref(oh), ctypes.byref(ow))
            assert lp and oh.value == H // 16 and ow.value == W // 16
            g[f"encode_{H}x{W}"] = np.ctypeslib.as_array(lp, shape=(128, oh.value, ow.value)).copy()
            libc.free(ctypes.cast(lp, vp))
            print("vae encode", H, W, "std", g[f"encode_{H}x{W}"].std(), flush=True)
        L.flux_vae_free(vae)
    return g


# shared with tests/test_oracle_golden.py: token ids and masks of the two encoder cases
QWEN3_CASES = {"masked8": ([151644, 872, 198, 64, 8251, 151645, 151643, 151643], [1, 1, 1, 1, 1, 1, 0, 0]),
               "plain5": ([11, 4999, 151935, 0, 77777], None)}


def qwen3_golden():
    """The reference's qwen3_forward (flux_qwen3.c:1041, CPU arm, weights streamed layer by layer through
    qwen3_model_load_mmap) on the synthetic full-size encoder of model_spec.make_qwen3_weights.
    Writes an 8 GB model directory under a temporary directory while it runs."""
    import tempfile
    g = {}
    L.qwen3_model_load_mmap.restype = vp
    L.qwen3_model_load_mmap.argtypes = [ctypes.c_char_p]
    L.qwen3_forward.restype = vp
    L.qwen3_forward.argtypes = [vp, vp, vp, c_i]
    L.qwen3_model_free.argtypes = [vp]
    cfg = QWEN3_4B
    with tempfile.TemporaryDirectory() as d:
        W = make_qwen3_weights(cfg)
        names = list(W)
        half = names.index("model.layers.18.input_layernorm.weight")
        write_safetensors(os.path.join(d, "model-00001-of-00002.safetensors"), {n: W[n] for n in names[:half]})
        write_safetensors(os.path.join(d, "model-00002-of-00002.safetensors"), {n: W[n] for n in names[half:]})
        del W
        m = L.qwen3_model_load_mmap(d.encode())
        assert m
        for key, (ids, mask) in QWEN3_CASES.items():
            ids = np.array(ids, np.int32)
            mk = None if mask is None else np.array(mask, np.int32)
            p = L.qwen3_forward(m, P(ids), None if mk is None else P(mk), ids.size)
            assert p
            out = np.ctypeslib.as_array(ctypes.cast(p, ctypes.POINTER(c_f)), shape=(ids.size * 3 * cfg.hidden,)).copy()
            ctypes.CDLL(None).free(ctypes.c_void_p(p))
            g[key] = out.reshape(ids.size, 3 * cfg.hidden)
            print("qwen3", key, "std", g[key].std(), flush=True)
        L.qwen3_model_free(m)
    return g


def full_c1(qk):
    """Config c1 of the benchmark at the real 4B architecture: 4x4 latent, 64 text tokens, t=1."""
    cfg = KLEIN_4B
    W = make_weights(cfg, 42, 0.02, qk)
    m = new_model(cfg, W)
    del W
    lat = normal_f32((cfg.channels, 4, 4), 42, 1000)
    txt = normal_f32((64, cfg.text_dim), 42, 1001)
    v = take(L.flux_transformer_forward(m, P(lat), 4, 4, P(txt), 64, 1.0), (cfg.channels, 4, 4))
    L.ref_model_free(m)
    return {"velocity": v}


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--full", action="store_true")
    ap.add_argument("--only-vae", action="store_true", help="rewrite vae.npz only")
    ap.add_argument("--qwen3", action="store_true", help="rewrite qwen3_4b.npz only (8 GB of temporary files, minutes)")
    args = ap.parse_args()
    L = load()
    if args.qwen3:
        np.savez_compressed(os.path.join(HERE, "qwen3_4b.npz"), **qwen3_golden())
        sys.exit(0)
    np.savez_compressed(os.path.join(HERE, "vae.npz"), **vae_golden())
    if args.only_vae:
        sys.exit(0)
    np.savez_compressed(os.path.join(HERE, "ops.npz"), **ops_golden())
    for qk in ("literal", "sharp"):
        np.savez_compressed(os.path.join(HERE, f"tiny_{qk}.npz"), **model_golden(TINY, qk))
    if args.full:
        for qk in ("literal", "sharp"):
            np.savez_compressed(os.path.join(HERE, f"klein4b_c1_{qk}.npz"), **full_c1(qk))
            print("wrote full c1", qk, flush=True)
    print("golden fixtures written to", HERE)
