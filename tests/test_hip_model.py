"""Whole-model parity of the HIP backend against the CPU oracle and the reference's golden vectors.

Gates (the stated tolerance of the backend): per-forward velocity relative L2 <= 2e-2 and
cosine >= 0.999 against the fp32 CPU path; final latent PSNR >= 35 dB (peak = range of the
reference latent).
"""
import os

import numpy as np
import pytest

from metrics import rel_l2, cosine, psnr
from model_spec import TINY, SMALL, KLEIN_4B, make_weights, normal_f32, write_safetensors

pytestmark = pytest.mark.gpu

REL_L2_MAX, COS_MIN, PSNR_MIN = 2e-2, 0.999, 35.0


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


# std 0.02 is the benchmark's literal initialisation; the larger values give the small models the
# per-layer gain the 4B model has at 0.02, so that attention and modulation shape the output
# (moving a reference image's RoPE offset then changes the velocity by 5-8 %).
@pytest.mark.parametrize("cfg,qk,std", [(TINY, "literal", 0.02), (TINY, "sharp", 0.02), (SMALL, "sharp", 0.02),
                                        (TINY, "sharp", 0.08), (SMALL, "sharp", 0.05)])
def test_forward_and_refs(hip, oracle_mod, cfg, qk, std):
    W = make_weights(cfg, 42, std, qk)
    o = oracle_mod.Oracle(cfg, W)
    m = hip.Transformer(cfg, W)
    lat = normal_f32((cfg.channels, 5, 7), 11, 1)
    txt = normal_f32((40, cfg.text_dim), 11, 2)
    r1 = (normal_f32((cfg.channels, 3, 4), 11, 3), 3, 4, 10)
    r2 = (normal_f32((cfg.channels, 2, 5), 11, 4), 2, 5, 20)
    gate(m.forward(lat, 5, 7, txt, 1.0), o.forward(lat, 5, 7, txt, 1.0), "no refs t=1")
    gate(m.forward(lat, 5, 7, txt, 0.3), o.forward(lat, 5, 7, txt, 0.3), "no refs t=0.3")
    gate(m.forward(lat, 5, 7, txt, 0.6, refs=[r1]), o.forward(lat, 5, 7, txt, 0.6, refs=[r1]), "one ref")
    gate(m.forward(lat, 5, 7, txt, 0.6, refs=[r1, r2]), o.forward(lat, 5, 7, txt, 0.6, refs=[r1, r2]), "two refs")
    m.close(); o.close()


def test_reference_golden_tiny(hip, golden_dir):
    """Straight against vectors the reference's own C code produced (tests/golden/make_golden.py)."""
    for qk in ("literal", "sharp"):
        g = np.load(os.path.join(golden_dir, f"tiny_{qk}.npz"))
        cfg = TINY
        m = hip.Transformer(cfg, make_weights(cfg, 42, 0.02, qk))
        lat = normal_f32((cfg.channels, 4, 4), 7, 100)
        txt = normal_f32((16, cfg.text_dim), 7, 101)
        txt_u = normal_f32((12, cfg.text_dim), 7, 102)
        r1 = (normal_f32((cfg.channels, 2, 3), 7, 103), 2, 3, 10)
        r2 = (normal_f32((cfg.channels, 3, 2), 7, 104), 3, 2, 20)
        gate(m.forward(lat, 4, 4, txt, 1.0), g["fwd_t1.0"], f"{qk} fwd t=1")
        gate(m.forward(lat, 4, 4, txt, 0.37), g["fwd_t0.37"], f"{qk} fwd t=0.37")
        gate(m.forward(lat, 4, 4, txt, 0.6, refs=[r1]), g["fwd_ref1"], f"{qk} one ref")
        gate(m.forward(lat, 4, 4, txt, 0.6, refs=[r1, r2]), g["fwd_ref2"], f"{qk} two refs")
        s3 = hip.schedule("official", 3, 16)
        for key, kw in (("euler3", {}), ("euler3_ref1", dict(refs=[r1])), ("euler3_ref2", dict(refs=[r1, r2]))):
            z = m.sample(lat, 4, 4, txt, s3, **kw)
            assert psnr(z, g[key]) >= PSNR_MIN, (key, psnr(z, g[key]))
        for key, kw in (("cfg2", {}), ("cfg2_ref1", dict(refs=[r1])), ("cfg2_ref2", dict(refs=[r1, r2]))):
            z = m.sample(lat, 4, 4, txt, s3[:3], txt_uncond=txt_u, guidance=4.0, **kw)
            assert psnr(z, g[key]) >= PSNR_MIN, (key, psnr(z, g[key]))
        m.close()


def test_sampler_trace_and_latent(hip, oracle_mod):
    """Per-step velocities and the final latent of a 4-step schedule, Euler and CFG + reference."""
    cfg = SMALL
    W = make_weights(cfg, 42, 0.02, "sharp")
    o = oracle_mod.Oracle(cfg, W)
    m = hip.Transformer(cfg, W)
    h, w = 6, 6
    z = normal_f32((cfg.channels, h, w), 12, 1)
    txt = normal_f32((48, cfg.text_dim), 12, 2)
    txt_u = normal_f32((48, cfg.text_dim), 12, 3)
    ref = (normal_f32((cfg.channels, h, w), 12, 4), h, w, 10)
    s = hip.schedule("official", 4, h * w)
    np.testing.assert_allclose(s, oracle_mod.official_schedule(4, h * w), atol=2e-7)
    zo, vo = o.sample_euler(z, h, w, txt, s, trace=True)
    zg, vg = m.sample(z, h, w, txt, s, trace=True)
    for i in range(4):
        gate(vg[i], vo[i], f"euler step {i}")
    assert psnr(zg, zo) >= PSNR_MIN, psnr(zg, zo)
    zo, vo = o.sample_euler_cfg(z, h, w, txt, txt_u, 4.0, s[:3], refs=[ref], trace=True)
    zg, vg = m.sample(z, h, w, txt, s[:3], refs=[ref], txt_uncond=txt_u, guidance=4.0, trace=True)
    for i in range(4):
        gate(vg[i], vo[i], f"cfg forward {i}")
    assert psnr(zg, zo) >= PSNR_MIN, psnr(zg, zo)
    m.close(); o.close()


def test_batched_cfg_equals_two_forwards(hip, oracle_mod):
    """A CFG step runs its unconditional and conditional forwards as one batch of two sequences (the default)
    or one after the other: same velocities up to GEMM tile/summation-order noise, and both within the gate
    of the oracle. Text lengths differ, and there are reference images, so every row offset is exercised."""
    cfg = SMALL
    W = make_weights(cfg, 42, 0.02, "sharp")
    o = oracle_mod.Oracle(cfg, W)
    m = hip.Transformer(cfg, W)
    h, w = 5, 7
    z = normal_f32((cfg.channels, h, w), 14, 1)
    txt = normal_f32((40, cfg.text_dim), 14, 2)
    txt_u = normal_f32((23, cfg.text_dim), 14, 3)
    refs = [(normal_f32((cfg.channels, 3, 4), 14, 4), 3, 4, 10), (normal_f32((cfg.channels, 2, 5), 14, 5), 2, 5, 20)]
    s = hip.schedule("official", 3, h * w)
    zo, vo = o.sample_euler_cfg(z, h, w, txt, txt_u, 3.5, s, refs=refs, trace=True)
    out = {}
    for on in (1, 0):
        hip.lib().flux_hip_set_batched_cfg(on)
        out[on] = m.sample(z, h, w, txt, s, refs=refs, txt_uncond=txt_u, guidance=3.5, trace=True)
    hip.lib().flux_hip_set_batched_cfg(1)
    for on in (1, 0):
        zg, vg = out[on]
        for i in range(6):
            gate(vg[i], vo[i], f"cfg forward {i} (batched={on})")
        assert psnr(zg, zo) >= PSNR_MIN
    assert rel_l2(out[1][1], out[0][1]) < 2e-3
    m.close(); o.close()


def test_single_stream_projection_as_one_or_two_launches(hip, oracle_mod):
    """A single-stream block's [Q | K | V | gate | up] projection runs as one launch (the default) or as two: both
    within the gate of the oracle, and equal up to the tile choice's summation order. 30 tokens (where the two
    launches run as K slices) and 300."""
    cfg = SMALL
    W = make_weights(cfg, 42, 0.05, "sharp")
    o = oracle_mod.Oracle(cfg, W)
    m = hip.Transformer(cfg, W)
    L = hip.lib()
    try:
        for h, w, nt in ((4, 5, 10), (16, 17, 28)):
            lat = normal_f32((cfg.channels, h, w), 19, 1)
            txt = normal_f32((nt, cfg.text_dim), 19, 2)
            want = o.forward(lat, h, w, txt, 0.6)
            got = {}
            for mode in (0, 1):
                L.flux_hip_set_fused_qkv_mlp(mode)
                got[mode] = m.forward(lat, h, w, txt, 0.6)
                gate(got[mode], want, f"{h}x{w}+{nt} tokens, fused projection mode {mode}")
            assert rel_l2(got[1], got[0]) < 5e-3      # bf16 intermediates round differently when the K slices of the two-launch form sum in another order
    finally:
        L.flux_hip_set_fused_qkv_mlp(1)
    m.close(); o.close()


def test_broken_rope_would_be_caught(hip, oracle_mod):
    """Sensitivity check: against an oracle whose image RoPE is mirrored the gate must fail,
    otherwise the sharp fixture would say nothing about RoPE in the HIP kernels."""
    cfg = TINY
    W = make_weights(cfg, 42, 0.08, "sharp")     # weights large enough for attention to matter
    o = oracle_mod.Oracle(cfg, W)
    m = hip.Transformer(cfg, W)
    lat = normal_f32((cfg.channels, 6, 6), 13, 1)
    txt = normal_f32((24, cfg.text_dim), 13, 2)
    good = o.forward(lat, 6, 6, txt, 0.8)
    wrong = o.forward(lat.reshape(cfg.channels, 6, 6).transpose(0, 2, 1).copy(), 6, 6, txt, 0.8)  # rows<->cols
    wrong = wrong.transpose(0, 2, 1)
    got = m.forward(lat, 6, 6, txt, 0.8)
    gate(got, good, "correct rope")
    assert rel_l2(got, wrong) > 3 * REL_L2_MAX, rel_l2(got, wrong)
    # same for the T axis of a reference image: offsets 10 and 20 must be told apart
    ref = normal_f32((cfg.channels, 6, 6), 13, 3)
    good = o.forward(lat, 6, 6, txt, 0.8, refs=[(ref, 6, 6, 10)])
    wrong = o.forward(lat, 6, 6, txt, 0.8, refs=[(ref, 6, 6, 20)])
    got = m.forward(lat, 6, 6, txt, 0.8, refs=[(ref, 6, 6, 10)])
    gate(got, good, "ref offset 10")
    assert rel_l2(got, wrong) > 2 * REL_L2_MAX, rel_l2(got, wrong)
    m.close(); o.close()


def test_safetensors_file_loader(hip, oracle_mod, tmp_path):
    cfg = TINY
    W = make_weights(cfg, 42, 0.02, "sharp")
    p = tmp_path / "tiny.safetensors"
    write_safetensors(str(p), W)
    a = hip.Transformer(cfg, path=str(p))
    b = hip.Transformer(cfg, W)
    lat = normal_f32((cfg.channels, 4, 4), 14, 1)
    txt = normal_f32((16, cfg.text_dim), 14, 2)
    assert np.array_equal(a.forward(lat, 4, 4, txt, 0.5), b.forward(lat, 4, 4, txt, 0.5))
    a.close(); b.close()
    # a file with a tensor missing must be refused, not half-loaded
    W.pop("proj_out.weight")
    write_safetensors(str(p), W)
    with pytest.raises(hip.FluxHipError):
        hip.Transformer(cfg, path=str(p))


def test_malformed_weight_files_are_refused(hip, tmp_path):
    """Every way a .safetensors file can lie about itself ends in an error with a reason, never in a read
    outside the mapping; tensors of other types or names are passed over."""
    import json
    import struct
    cfg = TINY
    W = make_weights(cfg, 42, 0.02, "sharp")
    good = tmp_path / "good.safetensors"
    write_safetensors(str(good), W)
    raw = good.read_bytes()
    hlen = struct.unpack("<Q", raw[:8])[0]
    header, data = json.loads(raw[8:8 + hlen]), raw[8 + hlen:]

    def write(name, hdr, payload=data, hlen_override=None):
        hj = json.dumps(hdr, separators=(",", ":")).encode() if isinstance(hdr, dict) else hdr
        q = tmp_path / name
        q.write_bytes(struct.pack("<Q", len(hj) if hlen_override is None else hlen_override) + hj + payload)
        return str(q)

    def altered(fn):
        h = json.loads(json.dumps(header))
        fn(h)
        return h

    first = next(iter(header))
    bad = {
        "truncated data": write("a.safetensors", header, data[:len(data) // 2]),
        "header length beyond the file": write("b.safetensors", header, hlen_override=1 << 40),
        "header length zero": write("c.safetensors", header, hlen_override=0),
        "not JSON": write("d.safetensors", b"[1, 2, 3]" + b" " * 7),
        "cut-off JSON": write("e.safetensors", json.dumps(header).encode()[:hlen // 2]),
        "shape larger than the byte range": write("f.safetensors", altered(lambda h: h[first].update(shape=[h[first]["shape"][0] * 2] + h[first]["shape"][1:]))),
        "shape that overflows": write("g.safetensors", altered(lambda h: h[first].update(shape=[1 << 39, 1 << 39]))),
        "offsets reversed": write("h.safetensors", altered(lambda h: h[first].update(data_offsets=h[first]["data_offsets"][::-1]))),
        "offsets beyond the data": write("i.safetensors", altered(lambda h: h[first].update(data_offsets=[len(data), len(data) + h[first]["data_offsets"][1]]))),
        "no offsets": write("j.safetensors", altered(lambda h: h[first].pop("data_offsets"))),
    }
    (tmp_path / "k.safetensors").write_bytes(b"abc")
    bad["shorter than its length field"] = str(tmp_path / "k.safetensors")
    bad["missing file"] = str(tmp_path / "nothing.safetensors")
    for what, path in bad.items():
        with pytest.raises(hip.FluxHipError) as err:
            hip.Transformer(cfg, path=path)
        print(f"{what}: {err.value}", flush=True)
        assert len(str(err.value)) > 20
    # passed over: a tensor of a type the library has no use for, and one under a name it does not know
    extra = altered(lambda h: (h.update({"step_count": {"dtype": "I64", "shape": [1], "data_offsets": [len(data), len(data) + 8]}}),
                               h.update({"ema.decay": {"dtype": "BF16", "shape": [4], "data_offsets": [len(data) + 8, len(data) + 16]}}),
                               h.update({"__metadata__": {"format": "pt"}})))
    extra_path = write("l.safetensors", extra, data + bytes(16))
    a = hip.Transformer(cfg, path=extra_path)
    b = hip.Transformer(cfg, path=str(good))
    lat = normal_f32((cfg.channels, 4, 4), 14, 1)
    txt = normal_f32((16, cfg.text_dim), 14, 2)
    want = b.forward(lat, 4, 4, txt, 0.5)
    assert np.array_equal(a.forward(lat, 4, 4, txt, 0.5), want)
    a.close(); b.close()
    # the same file through the handle the reference's own parser makes of it (its dtype numbering goes on past
    # BF16: I32 = 3, I64 = 4, BOOL = 5, flux_safetensors.h:20-28): the I64 entry is passed over there too
    import ctypes
    ref_so = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "oracle", "_ref", "libfluxref.so")
    if os.path.exists(ref_so):
        R = ctypes.CDLL(os.path.realpath(ref_so))
        R.safetensors_open.restype = ctypes.c_void_p
        R.safetensors_open.argtypes = [ctypes.c_char_p]
        sf = R.safetensors_open(extra_path.encode())
        assert sf
        L = hip.lib()
        L.flux_transformer_load_safetensors_mmap.restype = ctypes.c_void_p
        L.flux_transformer_load_safetensors_mmap.argtypes = [ctypes.c_void_p]
        tf = L.flux_transformer_load_safetensors_mmap(sf)
        assert tf, L.flux_hip_last_error()
        p = L.flux_transformer_forward(tf, lat.ctypes.data, 4, 4, txt.ctypes.data, 16, ctypes.c_float(0.5))
        assert p, L.flux_hip_last_error()
        got = np.ctypeslib.as_array(ctypes.cast(p, ctypes.POINTER(ctypes.c_float)), shape=(cfg.channels * 16,)).copy()
        hip.libc_free(p)
        L.flux_transformer_free(tf)            # closes the handle it took over
        assert np.array_equal(got.reshape(want.shape), want)


def test_error_paths(hip):
    cfg = TINY
    m = hip.Transformer(cfg)          # no weights yet
    lat = normal_f32((cfg.channels, 2, 2), 15, 1)
    txt = normal_f32((8, cfg.text_dim), 15, 2)
    with pytest.raises(hip.FluxHipError):
        m.forward(lat, 2, 2, txt, 0.5)
    with pytest.raises(hip.FluxHipError):
        m.set_tensor("proj_out.weight", np.zeros(3, np.uint16))        # wrong size
    with pytest.raises(hip.FluxHipError):
        m.set_tensor("no.such.tensor", np.zeros(3, np.uint16))
    m.close()


def test_sequence_growth_between_calls(hip, oracle_mod):
    """Work buffers and RoPE tables are re-made when the token count grows or shrinks."""
    cfg = TINY
    W = make_weights(cfg, 42, 0.02, "sharp")
    o = oracle_mod.Oracle(cfg, W)
    m = hip.Transformer(cfg, W)
    for (h, w, nt) in ((2, 2, 8), (9, 11, 70), (3, 3, 5), (9, 11, 70)):
        lat = normal_f32((cfg.channels, h, w), 16, h * 100 + w)
        txt = normal_f32((nt, cfg.text_dim), 16, nt)
        gate(m.forward(lat, h, w, txt, 0.7), o.forward(lat, h, w, txt, 0.7), f"{h}x{w}+{nt}")
    m.close(); o.close()


@pytest.mark.parametrize("qk", ["literal", "sharp"])
def test_klein4b_c1_against_reference_golden(hip, golden_dir, qk):
    """Real 4B architecture, 4x4 latent + 64 text tokens, t = 1: the velocity the reference's C
    code computed for the same seeded weights and inputs (fixture written by make_golden.py --full)."""
    g = np.load(os.path.join(golden_dir, f"klein4b_c1_{qk}.npz"))
    cfg = KLEIN_4B
    m = hip.Transformer(cfg)
    from model_spec import tensor_shapes
    for name in tensor_shapes(cfg):            # one tensor at a time keeps the host footprint small
        m.set_tensor(name, make_weights(cfg, 42, 0.02, qk, only=[name])[name])
    lat = normal_f32((cfg.channels, 4, 4), 42, 1000)
    txt = normal_f32((64, cfg.text_dim), 42, 1001)
    gate(m.forward(lat, 4, 4, txt, 1.0), g["velocity"], f"4B c1 {qk}")
    m.close()


def test_long_ragged_sequence(hip, oracle_mod):
    """8000 image tokens (100 x 80, beyond the 1024^2 case) + 333 text tokens on the small model:
    many 256-wide tiles, a ragged tail in every kernel, the 256-query attention workgroups."""
    cfg = SMALL
    W = make_weights(cfg, 42, 0.05, "sharp")
    o = oracle_mod.Oracle(cfg, W)
    m = hip.Transformer(cfg, W)
    lat = normal_f32((cfg.channels, 100, 80), 17, 1)
    txt = normal_f32((333, cfg.text_dim), 17, 2)
    gate(m.forward(lat, 100, 80, txt, 0.9), o.forward(lat, 100, 80, txt, 0.9), "100x80 + 333")
    m.close(); o.close()


def test_reference_loader_entry_point(hip, golden_dir, tmp_path):
    """flux_transformer_load_safetensors_mmap() fed with the handle the reference's own
    safetensors_open() returns (its C code compiled in place, oracle/_ref): checks the mirrored
    struct layout, the name mapping and ownership on the real 4B file layout."""
    import ctypes
    ref_so = os.path.join(os.path.dirname(golden_dir), "..", "oracle", "_ref", "libfluxref.so")
    if not os.path.exists(ref_so):
        pytest.skip("oracle/_ref/libfluxref.so is not built")
    from model_spec import tensor_shapes
    cfg = KLEIN_4B
    path = "/dev/shm/flux_hip_test_4b.safetensors" if os.path.isdir("/dev/shm") else str(tmp_path / "m.safetensors")
    try:
        # stream the 7.75 GB file tensor by tensor
        import json
        shapes = tensor_shapes(cfg)
        header, off = {}, 0
        for name, shp in shapes.items():
            nb = int(np.prod(shp)) * 2
            header[name] = {"dtype": "BF16", "shape": list(shp), "data_offsets": [off, off + nb]}
            off += nb
        hj = json.dumps(header, separators=(",", ":")).encode()
        hj += b" " * ((8 - len(hj) % 8) % 8)
        with open(path, "wb") as f:
            f.write(len(hj).to_bytes(8, "little"))
            f.write(hj)
            for name in shapes:
                f.write(make_weights(cfg, 42, 0.02, "sharp", only=[name])[name].tobytes())
        R = ctypes.CDLL(os.path.realpath(ref_so))
        R.safetensors_open.restype = ctypes.c_void_p
        R.safetensors_open.argtypes = [ctypes.c_char_p]
        sf = R.safetensors_open(path.encode())
        assert sf
        L = hip.lib()
        L.flux_transformer_load_safetensors_mmap.restype = ctypes.c_void_p
        L.flux_transformer_load_safetensors_mmap.argtypes = [ctypes.c_void_p]
        tf = L.flux_transformer_load_safetensors_mmap(sf)
        assert tf, L.flux_hip_last_error()
        lat = normal_f32((cfg.channels, 4, 4), 42, 1000)
        txt = normal_f32((64, cfg.text_dim), 42, 1001)
        p = L.flux_transformer_forward(tf, lat.ctypes.data, 4, 4, txt.ctypes.data, 64, 1.0)
        assert p, L.flux_hip_last_error()
        v = np.ctypeslib.as_array(ctypes.cast(p, ctypes.POINTER(ctypes.c_float)), shape=(cfg.channels * 16,)).copy()
        hip.libc_free(p)
        g = np.load(os.path.join(golden_dir, "klein4b_c1_sharp.npz"))
        gate(v, g["velocity"], "4B c1 through the reference loader entry point")
        L.flux_transformer_free(tf)      # also closes sf (mmap mode owns the handle)
    finally:
        if os.path.exists(path):
            os.remove(path)


def test_callbacks_fire_in_order(hip):
    """Step, sub-step and progress callbacks (flux_kernels.h:245-256, flux_sample.c:240,254) fire on
    the calling thread in the reference's order."""
    import ctypes
    cfg = TINY
    m = hip.Transformer(cfg, make_weights(cfg, 42, 0.02, "sharp"))
    L = hip.lib()
    log = []
    STEP = ctypes.CFUNCTYPE(None, ctypes.c_int, ctypes.c_int)
    SUB = ctypes.CFUNCTYPE(None, ctypes.c_int, ctypes.c_int, ctypes.c_int)
    step_cb = STEP(lambda s, n: log.append(("step", s, n)))
    sub_cb = SUB(lambda t, i, n: log.append(("sub", t, i, n)))
    prog_cb = STEP(lambda s, n: log.append(("progress", s, n)))
    ctypes.c_void_p.in_dll(L, "flux_step_callback").value = ctypes.cast(step_cb, ctypes.c_void_p).value
    ctypes.c_void_p.in_dll(L, "flux_substep_callback").value = ctypes.cast(sub_cb, ctypes.c_void_p).value
    try:
        z = normal_f32((cfg.channels, 2, 2), 18, 1)
        txt = normal_f32((8, cfg.text_dim), 18, 2)
        sched = hip.schedule("linear", 2)
        L.flux_sample_euler.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int] * 4 + [ctypes.c_void_p, ctypes.c_int,
                                                                                     ctypes.c_void_p, ctypes.c_int, STEP]
        p = L.flux_sample_euler(m.h, None, z.ctypes.data, 1, cfg.channels, 2, 2, txt.ctypes.data, 8,
                                sched.ctypes.data, 2, prog_cb)
        assert p
        hip.libc_free(p)
        # a single forward (flux_transformer.c:3115) fires the block callbacks only and ADDS to the stage timers
        sampler_log, log[:] = list(log), []
        total = ctypes.c_double.in_dll(L, "flux_timing_transformer_total")
        t0 = total.value
        m.forward(z, 2, 2, txt, 0.5)
        t1 = total.value
        m.forward(z, 2, 2, txt, 0.5)
        assert t0 > 0 and t1 > t0 and total.value > t1
        forward_log, log[:] = list(log), sampler_log
    finally:
        ctypes.c_void_p.in_dll(L, "flux_step_callback").value = None
        ctypes.c_void_p.in_dll(L, "flux_substep_callback").value = None
    per_step = [("sub", 0, i, cfg.n_double) for i in range(cfg.n_double)] + \
               [("sub", 1, i, cfg.n_single) for i in range(cfg.n_single)] + [("sub", 2, 0, 1)]
    want = []
    for s in (1, 2):
        want += [("step", s, 2)] + per_step + [("progress", s, 2)]
    assert log == want
    assert forward_log == per_step + per_step
    m.close()
