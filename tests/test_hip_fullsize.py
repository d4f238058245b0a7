"""Parity at the benchmark's real shapes: FLUX.2-klein-4B architecture, random-init bf16 weights
N(0, 0.02) seed 42, against the fp32 CPU oracle on the same inputs.

c2: 256 image + 512 text tokens, full 4-step distilled schedule (velocities + final latent)
c3: 1024 + 512 tokens, first step of the 4-step schedule (sharp weights, see below)
c4: 4096 + 512 tokens (headline shape), full 4-step schedule
c5: CFG + one reference image, (1024 + 1024) + 512 tokens, first two steps of the 50-step schedule = four forwards
    (flux_sample.c:534-590): the unconditional and the conditional velocity of each step and the guided velocity
    vu + 4 (vc - vu) that moves the latent, in which the two forwards' errors can add up to seven-fold
Gates: velocity rel-L2 <= 2e-2, cosine >= 0.999, latent PSNR >= 35 dB. Where a run covers only the first steps of a
schedule the latent barely moves (the 50-step schedule's first dt is -0.0037: any velocity would pass a PSNR on the
latent), so there the PSNR is taken on the displacement z - z0, peak = the range of the oracle's displacement.

Two weight sets. "literal": every tensor N(0, 0.02), the QK-norm weights included; attention logits
are then of order 1e-4, the softmax is uniform and an error in RoPE, QK-norm or softmax cannot move
the velocity beyond the gate. "sharp": the same tensors with the QK-norm weights at 1.0 (logits of
order one); c3, c4 and c5 run their first step with it as well, and a control shows that an oracle
whose image RoPE axes are swapped fails the gate there (flux_transformer.c:719-741, 1052-1106,
1335-1460 are what these cases can see and the literal ones cannot).
"""
import numpy as np
import pytest

from metrics import rel_l2, cosine, psnr
from model_spec import KLEIN_4B, tensor_shapes, make_weights, normal_f32, is_qk_norm

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def models(oracle_mod):
    import fluxhip
    fluxhip.init()
    fluxhip.lib().flux_hip_linear_force_tile(-1)
    cfg = KLEIN_4B
    hip_m = fluxhip.Transformer(cfg)
    ora = oracle_mod.Oracle(cfg, {})
    for name in tensor_shapes(cfg):                      # one tensor at a time on the host
        a = make_weights(cfg, 42, 0.02, "literal", only=[name])[name]
        hip_m.set_tensor(name, a)
        rc = oracle_mod.lib().fo_model_set_bf16(ora.h, name.encode(), a.ctypes.data, a.size)
        assert rc == 0, name
    yield fluxhip, hip_m, ora
    hip_m.close()
    ora.close()


def set_qk_norm(models, oracle_mod, mode):
    """Replaces the QK-norm weights of both models: "literal" = N(0, 0.02), "sharp" = 1.0."""
    _, hip_m, ora = models
    for name in tensor_shapes(KLEIN_4B):
        if is_qk_norm(name):
            a = make_weights(KLEIN_4B, 42, 0.02, mode, only=[name])[name]
            hip_m.set_tensor(name, a)
            assert oracle_mod.lib().fo_model_set_bf16(ora.h, name.encode(), a.ctypes.data, a.size) == 0


@pytest.fixture
def sharp(models, oracle_mod):
    set_qk_norm(models, oracle_mod, "sharp")
    yield
    set_qk_norm(models, oracle_mod, "literal")


def check(vg, vo, what):
    r, c = rel_l2(vg, vo), cosine(vg, vo)
    print(f"{what}: rel_l2={r:.3e} cos={c:.6f}", flush=True)
    assert r <= 2e-2 and c >= 0.999, (what, r, c)


def test_c2_full_schedule(models):
    fluxhip, m, o = models
    h = w = 16
    z = normal_f32((128, h, w), 123, 1)
    txt = normal_f32((512, 7680), 123, 2)
    s = fluxhip.schedule("official", 4, h * w)
    zo, vo = o.sample_euler(z, h, w, txt, s, trace=True)
    zg, vg = m.sample(z, h, w, txt, s, trace=True)
    for i in range(4):
        check(vg[i], vo[i], f"c2 step {i}")
    p = psnr(zg, zo)
    print(f"c2 final latent PSNR {p:.1f} dB", flush=True)
    assert p >= 35.0


def check_displacement(zg, zo, z0, what):
    """PSNR of what the steps did to the latent (z - z0), not of the latent: a run over the first steps of a schedule
    leaves z within a few per cent of z0 whatever the velocities were."""
    p = psnr(zg - z0, zo - z0)
    print(f"{what}: displacement PSNR {p:.1f} dB (latent PSNR {psnr(zg, zo):.1f} dB)", flush=True)
    assert p >= 35.0, (what, p)


def first_step(models, name, h, w):
    fluxhip, m, o = models
    z = normal_f32((128, h, w), 123, 1)
    txt = normal_f32((512, 7680), 123, 2)
    s = fluxhip.schedule("official", 4, h * w)[:2]
    zo, vo = o.sample_euler(z, h, w, txt, s, trace=True)
    zg, vg = m.sample(z, h, w, txt, s, trace=True)
    check(vg[0], vo[0], f"{name} step 0")
    check_displacement(zg, zo, z, name)
    return z, txt, s, vg[0], vo[0]


def test_c4_full_schedule(models):
    """The headline shape through all four steps of its schedule: every step's velocity and the final latent."""
    fluxhip, m, o = models
    h = w = 64
    z = normal_f32((128, h, w), 123, 1)
    txt = normal_f32((512, 7680), 123, 2)
    s = fluxhip.schedule("official", 4, h * w)
    zo, vo = o.sample_euler(z, h, w, txt, s, trace=True)
    zg, vg = m.sample(z, h, w, txt, s, trace=True)
    for i in range(4):
        check(vg[i], vo[i], f"c4 step {i}")
    p = psnr(zg, zo)
    print(f"c4 final latent PSNR {p:.1f} dB", flush=True)
    assert p >= 35.0


def test_c3_sharp_first_step_and_rope_control(models, sharp):
    """QK-norm weights of 1.0: RoPE, QK-norm and softmax decide the output (24 heads x 1536 tokens). Against an oracle
    whose image rows and columns are swapped the same velocity must FAIL the gate; if it passed, this fixture
    would say nothing about the attention side either."""
    fluxhip, m, o = models
    z, txt, s, vg, vo = first_step(models, "c3 sharp", 32, 32)
    h = w = 32
    zt = z.reshape(128, h, w).transpose(0, 2, 1).copy()
    _, vw = o.sample_euler(zt, h, w, txt, s, trace=True)
    wrong = vw[0].reshape(128, h, w).transpose(0, 2, 1).ravel()
    r = rel_l2(vg, wrong)
    print(f"c3 sharp against the mirrored oracle: rel_l2={r:.3e}", flush=True)
    assert r > 2 * 2e-2, r          # measured: 5.4e-2, seven times the error of the right answer


def test_c4_sharp_first_step(models, sharp):
    """24 heads x 4608 tokens with logits of order one: the 256-query workgroups and the head order over the XCDs."""
    first_step(models, "c4 sharp", 64, 64)


def c5_steps(models, what, steps):
    """The first `steps` steps of c5: per step the unconditional and the conditional velocity, and the guided velocity
    v = vu + g (vc - vu) with g = 4 (flux_sample.c:575-581), which is what the Euler update applies."""
    fluxhip, m, o = models
    h = w = 32
    g = 4.0
    z = normal_f32((128, h, w), 123, 1)
    txt = normal_f32((512, 7680), 123, 2)
    txt_u = normal_f32((512, 7680), 123, 3)
    ref = (normal_f32((128, h, w), 123, 10), h, w, 10)
    s = fluxhip.schedule("official", 50, h * w)[:steps + 1]
    zo, vo = o.sample_euler_cfg(z, h, w, txt, txt_u, g, s, refs=[ref], trace=True)
    zg, vg = m.sample(z, h, w, txt, s, refs=[ref], txt_uncond=txt_u, guidance=g, trace=True)
    for i in range(steps):
        check(vg[2 * i], vo[2 * i], f"{what} step {i} uncond")
        check(vg[2 * i + 1], vo[2 * i + 1], f"{what} step {i} cond")
        # The guided velocity is 4 vc - 3 vu, so its error is 4 ec - 3 eu: between one and seven times a forward's
        # error, depending on how the two forwards' rounding errors correlate. They hardly do (the two sequences'
        # activations differ from the first joint attention on, by far more than a bf16 step), and on this fixture
        # vc - vu is a few per cent of v, so the guided velocity is about v and its error about five forwards' errors
        # in quadrature: 3.2e-2 measured for 7.6e-3 per forward. That is beyond the 2e-2 asked of a velocity and is what
        # bf16 operands allow here; the gate below is 5 x 8e-3, which a systematic fault (wrong text, swapped passes,
        # wrong guidance weight: errors of order |vc - vu| x g and more) still misses by far.
        gg, go = vg[2 * i] + g * (vg[2 * i + 1] - vg[2 * i]), vo[2 * i] + g * (vo[2 * i + 1] - vo[2 * i])
        eu, ec = (vg[2 * i] - vo[2 * i]).astype(np.float64), (vg[2 * i + 1] - vo[2 * i + 1]).astype(np.float64)
        rho = float(eu.dot(ec) / (np.linalg.norm(eu) * np.linalg.norm(ec)))
        r, c = rel_l2(gg, go), cosine(gg, go)
        print(f"{what} step {i} guided: rel_l2={r:.3e} cos={c:.6f}; |vc - vu| / |vu| = {rel_l2(vo[2 * i + 1], vo[2 * i]):.3e}, "
              f"correlation of the two forwards' errors {rho:.3f}", flush=True)
        assert r <= 4e-2 and c >= 0.999, (what, i, r, c)
    # the trace holds what the update used: z must be z0 + sum dt_i * guided_i on both sides
    disp = sum((s[i + 1] - s[i]) * (vo[2 * i] + g * (vo[2 * i + 1] - vo[2 * i])) for i in range(steps))
    assert rel_l2(zo.ravel() - z.ravel(), disp) < 1e-4
    check_displacement(zg, zo, z, what)


def test_c5_cfg_with_reference_two_steps(models):
    c5_steps(models, "c5", 2)


def test_c5_sharp_cfg_with_reference_first_step(models, sharp):
    """Batched CFG (two sequences, per-sequence K / V^T offsets) and the reference image's T offset with sharp logits."""
    c5_steps(models, "c5 sharp", 1)


def test_maximum_size_properties(models):
    """1792 x 1792 (12544 image + 512 text tokens, the largest image the reference accepts, flux.h:52), alone
    and with two reference images of other sizes (14244 tokens): the oracle would need half an hour per
    forward, so only what does not depend on it - finite velocities of unit scale, the same bits on a second run."""
    fluxhip, m, _ = models
    for h, w, nt, refs in ((112, 112, 512, []), (112, 109, 300, [(40, 37, 10), (16, 16, 20)])):
        z = normal_f32((128, h, w), 124, 1)
        txt = normal_f32((nt, 7680), 124, 2)
        rf = [(normal_f32((128, rh, rw), 124, 10 + i), rh, rw, t) for i, (rh, rw, t) in enumerate(refs)]
        s = fluxhip.schedule("official", 4, h * w)[:2]
        z1, v1 = m.sample(z, h, w, txt, s, refs=rf, trace=True)
        z2, v2 = m.sample(z, h, w, txt, s, refs=rf, trace=True)
        assert v1[0].shape == (128 * h * w,) and np.isfinite(v1[0]).all() and 0.3 < v1[0].std() < 3.0
        np.testing.assert_array_equal(v1[0], v2[0])
        np.testing.assert_array_equal(z1, z2)
