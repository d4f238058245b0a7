"""Heun and noise-injecting samplers, flux_generate_latent and the intermediate-image hook of the
HIP backend, against the CPU oracle and the reference's golden vectors. Same gates as the whole-
model tests: velocity rel-L2 <= 2e-2, cosine >= 0.999, final latent PSNR >= 35 dB.
"""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from metrics import rel_l2, cosine, psnr
from model_spec import TINY, SMALL, make_weights, normal_f32

pytestmark = pytest.mark.gpu

REL_L2_MAX, COS_MIN, PSNR_MIN = 2e-2, 0.999, 35.0
HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def hip():
    import fluxhip
    fluxhip.init()
    fluxhip.lib().flux_hip_linear_force_tile(-1)
    return fluxhip


def gate(got, want, what=""):
    r, c = rel_l2(got, want), cosine(got, want)
    print(f"{what}: rel_l2={r:.3e} cos={c:.6f}", flush=True)
    assert r <= REL_L2_MAX and c >= COS_MIN, (what, r, c)


def test_heun_and_ancestral_against_oracle(hip, oracle_mod):
    cfg = SMALL
    W = make_weights(cfg, 42, 0.05, "sharp")
    o = oracle_mod.Oracle(cfg, W)
    m = hip.Transformer(cfg, W)
    h, w = 5, 7
    z = normal_f32((cfg.channels, h, w), 21, 1)
    txt = normal_f32((40, cfg.text_dim), 21, 2)
    s = hip.schedule("sigmoid", 4, 0.5)
    np.testing.assert_allclose(s, oracle_mod.sigmoid_schedule(4, 0.5), atol=6e-7)

    zo, vo = o.sample_heun(z, h, w, txt, s, trace=True)
    zg, vg = m.sample_heun(z, h, w, txt, s, trace=True)
    assert vg.shape == vo.shape == (7, cfg.channels * h * w)
    for i in range(7):
        gate(vg[i], vo[i], f"heun forward {i}")
    assert psnr(zg, zo) >= PSNR_MIN, psnr(zg, zo)
    # second order really is in effect: the Euler result on the same schedule is measurably different
    ze = m.sample(z, h, w, txt, s)
    assert rel_l2(ze, zo) > 10 * rel_l2(zg, zo)

    zo, vo = o.sample_euler_ancestral(z, h, w, txt, s, 0.6, seed=2024, trace=True)
    zg, vg = m.sample_ancestral(z, h, w, txt, s, 0.6, seed=2024, trace=True)
    for i in range(4):
        gate(vg[i], vo[i], f"ancestral step {i}")
    assert psnr(zg, zo) >= PSNR_MIN, psnr(zg, zo)
    # a different noise stream gives a different latent; eta = 0 is the Euler sampler
    z2 = m.sample_ancestral(z, h, w, txt, s, 0.6, seed=2025)
    assert psnr(z2, zo) < 30.0
    assert np.array_equal(m.sample_ancestral(z, h, w, txt, s, 0.0), ze)
    m.close(); o.close()


def test_heun_and_ancestral_reference_golden(hip, golden_dir):
    """Against latents the reference's own samplers produced (tests/golden/make_golden.py: generator
    seeded with 99 right before the noise-injecting sampler, eta 0.7)."""
    import ctypes
    for qk in ("literal", "sharp"):
        g = np.load(os.path.join(golden_dir, f"tiny_{qk}.npz"))
        cfg = TINY
        m = hip.Transformer(cfg, make_weights(cfg, 42, 0.02, qk))
        lat = normal_f32((cfg.channels, 4, 4), 7, 100)
        txt = normal_f32((16, cfg.text_dim), 7, 101)
        s3 = hip.schedule("official", 3, 16)
        for key, z in (("heun3", m.sample_heun(lat, 4, 4, txt, s3)),
                       ("heun1", m.sample_heun(lat, 4, 4, txt, s3[:2])),
                       ("ancestral3", m.sample_ancestral(lat, 4, 4, txt, s3, 0.7, seed=99)),
                       ("ancestral3_eta0", m.sample_ancestral(lat, 4, 4, txt, s3, 0.0))):
            assert psnr(z, g[key]) >= PSNR_MIN, (qk, key, psnr(z, g[key]))
        # the entry points with the reference's names and argument order
        L = hip.lib()
        L.flux_rng_seed(99)
        p = L.flux_sample_euler_ancestral(m.h, lat.ctypes.data, 1, cfg.channels, 4, 4, txt.ctypes.data, 16,
                                          s3.ctypes.data, 3, 0.7, None)
        assert p
        za = np.ctypeslib.as_array(ctypes.cast(p, ctypes.POINTER(ctypes.c_float)), shape=(cfg.channels * 16,)).copy()
        hip.libc_free(p)
        assert psnr(za.reshape(cfg.channels, 4, 4), g["ancestral3"]) >= PSNR_MIN
        p = L.flux_sample_heun(m.h, lat.ctypes.data, 1, cfg.channels, 4, 4, txt.ctypes.data, 16, s3.ctypes.data, 3, None)
        assert p
        zh = np.ctypeslib.as_array(ctypes.cast(p, ctypes.POINTER(ctypes.c_float)), shape=(cfg.channels * 16,)).copy()
        hip.libc_free(p)
        assert psnr(zh.reshape(cfg.channels, 4, 4), g["heun3"]) >= PSNR_MIN
        assert not L.flux_sample_heun(m.h, lat.ctypes.data, 2, cfg.channels, 4, 4, txt.ctypes.data, 16, s3.ctypes.data, 3, None)
        assert b"batch" in L.flux_hip_last_error()
        m.close()


def test_generate_latent(hip, oracle_mod):
    """flux_generate_latent = flux_init_noise + linear schedule + Euler sampler (flux_sample.c:891-919)."""
    import ctypes
    cfg = TINY
    W = make_weights(cfg, 42, 0.05, "sharp")
    o = oracle_mod.Oracle(cfg, W)
    m = hip.Transformer(cfg, W)
    txt = normal_f32((20, cfg.text_dim), 22, 1)
    L = hip.lib()
    p = L.flux_generate_latent(m.h, txt.ctypes.data, 20, 96, 64, 3, 77, None)      # 6 x 4 latent
    assert p, L.flux_hip_last_error()
    zg = np.ctypeslib.as_array(ctypes.cast(p, ctypes.POINTER(ctypes.c_float)), shape=(cfg.channels, 6, 4)).copy()
    hip.libc_free(p)
    z0 = oracle_mod.init_noise(cfg.channels, 6, 4, 77)
    zo = o.sample_euler(z0, 6, 4, txt, oracle_mod.linear_schedule(3))
    assert psnr(zg, zo) >= PSNR_MIN, psnr(zg, zo)
    assert not L.flux_generate_latent(m.h, txt.ctypes.data, 20, 8, 64, 3, 77, None)     # height below one latent row
    m.close(); o.close()


CHILD = r"""
import ctypes, json, os, sys
import numpy as np
shim = ctypes.CDLL(sys.argv[1], mode=ctypes.RTLD_GLOBAL)      # before the library: its weak references bind here
root = sys.argv[2]
for p in ("flux2.c_amd", "oracle", "tests"):
    sys.path.insert(0, os.path.join(root, p))
import fluxhip, oracle as O
from metrics import psnr
from model_spec import TINY, make_weights, normal_f32
fluxhip.init()
cfg = TINY
W = make_weights(cfg, 42, 0.05, "sharp")
m = fluxhip.Transformer(cfg, W)
o = O.Oracle(cfg, W)
z = normal_f32((cfg.channels, 3, 4), 23, 1)
txt = normal_f32((12, cfg.text_dim), 23, 2)
s = fluxhip.schedule("linear", 3)
quiet = m.sample(z, 3, 4, txt, s)                     # hook symbols present but not set: nothing happens
assert shim.shim_decodes() == 0
shim.shim_enable(1)
zg = m.sample(z, 3, 4, txt, s)
zh = m.sample_heun(z, 3, 4, txt, s)
shim.shim_enable(0)
shim.shim_latent.restype = ctypes.POINTER(ctypes.c_float)
n = cfg.channels * 12
lat = [np.ctypeslib.as_array(shim.shim_latent(i), shape=(n,)).copy() for i in range(shim.shim_decodes())]
zo, vo = o.sample_euler(z, 3, 4, txt, s, trace=True)
zi = z.reshape(-1).copy()
inter = []
for i in range(2):
    zi = zi + (s[i + 1] - s[i]) * vo[i]
    inter.append(zi.copy())
print(json.dumps({
    "decodes": shim.shim_decodes(), "frees": shim.shim_frees(), "calls": shim.shim_calls(),
    "steps": [[shim.shim_step(i), shim.shim_total(i)] for i in range(shim.shim_calls())],
    "psnr": [float(psnr(lat[i], inter[i])) for i in range(2)],
    "same_final": bool(np.array_equal(quiet, zg)),
}))
"""


def test_step_image_hook(tmp_path):
    """With the application's hook symbols present and set, every step but the last hands the current
    latent to the application's decoder and the image to its callback (flux_sample.c:258-266)."""
    root = os.path.dirname(HERE)
    so = str(tmp_path / "libstepshim.so")
    subprocess.run(["gcc", "-O1", "-fPIC", "-shared", "-o", so, os.path.join(HERE, "step_image_shim.c")], check=True)
    r = subprocess.run([sys.executable, "-c", CHILD, so, root], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    out = json.loads(r.stdout.strip().splitlines()[-1])
    # Euler run: steps 1 and 2 of 3; Heun run: the same two
    assert out["decodes"] == 4 and out["frees"] == 4 and out["calls"] == 4, out
    assert out["steps"] == [[1, 3], [2, 3], [1, 3], [2, 3]], out
    assert min(out["psnr"]) >= PSNR_MIN, out
    assert out["same_final"], out
