#!/usr/bin/env python3
"""Benchmark of the MI355X denoising-transformer backend: denoise steps/s on one GPU.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c4]

One "step" is every transformer forward of one Euler step plus the latent update, at the real
FLUX.2-klein-4B architecture with random-init bf16 weights ~N(0, 0.02) and N(0,1) inputs
(there are no model files or datasets here). Inputs are resident in HBM before the timed
region; the host only queues kernels. Prints ONE JSON line.

Also measured in the same run:
  roofline      the dominant kernel (the fused [Q|K|V|gate|up] projection of the single-stream blocks): HIP events on
                the backend's stream around every launch of it inside the timed region; also launched alone
  cpu_baseline  the CPU oracle (fp32, BLAS when available) on a bounded sample of the same
                workload: one whole forward at full shape after a small warm-up forward
  box           what this machine's matrix pipes sustain on their own (a register-resident MFMA loop on random bit
                patterns, right after the timed steps), and the step's TFLOP/s over it: boxes differ by several per cent

--workload vae_c2 | vae_c3 | vae_c4 measures the step after the sampling loop instead: one "step" is
one VAE decode of a 16/32/64-wide latent to a 256/512/1024-pixel image; vae_enc_c2 | vae_enc_c3 |
vae_enc_c4 the VAE encoder on a picture of those sizes (the input of image-to-image generation).
--workload qwen3 measures the step before the loop: one forward of the text encoder over 512 tokens.
--workload att_c2 | att_c3 | att_c4 | att_c5 measures the attention operator alone (Q/K preparation + attention) at
that workload's sequence length.
--workload att_c1 ... att_c5 also exist for the other sequence lengths; bw_c3 | bw_c4 time the bandwidth-bound kernels
(AdaLN, Q/K preparation) against a streaming yardstick.
--workload mfma_peak measures no part of the model: what the matrix pipes sustain on their own (the measured
peak beside the datasheet's 2.5 PFLOP/s); mfma_issue what another instruction between a lone wave's MFMAs costs them;
gemm_vs_lib the step's projection shapes as plain GEMMs against the vendor library behind torch.matmul.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "flux2.c_amd"))

import numpy as np  # noqa: E402

import fluxhip  # noqa: E402
from model_spec import KLEIN_4B, FluxConfig, tensor_shapes, make_weights, normal_f32, normal_bf16, flops_per_forward  # noqa: E402

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA peak (datasheet)
# Bytes per launch that the dominant kernel moves beyond its L2s: not measured in this run (it takes hardware counters) but
# taken from profiles/gemm_qkv_swiglu_c4_traffic.txt, i.e. from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# `bench.py --calibrate` on the kernel as it is in this tree, scaled by the same counters on a streaming kernel of known size.
# The figure follows from the tile walk (1189 MB of operand rows per launch by construction) and has not moved with the loop.
PEAK_HBM_GBPS = 8000.0      # MI355X HBM3E peak (datasheet)
TRAFFIC_BYTES = {("c4", True): 1_365_000_000}   # keyed by (workload, fused [Q|K|V|gate|up] launch); null where no profile covers the launch

# (latent h, w, text tokens, reference-image latents [(h, w, t_offset)], cfg, schedule steps)
WORKLOADS = {
    "c1": dict(h=4, w=4, txt=64, refs=[], cfg=False, desc="64x64: 16 image + 64 text tokens"),
    "c2": dict(h=16, w=16, txt=512, refs=[], cfg=False, desc="256x256: 256 image + 512 text tokens"),
    "c3": dict(h=32, w=32, txt=512, refs=[], cfg=False, desc="512x512: 1024 image + 512 text tokens"),
    "c4": dict(h=64, w=64, txt=512, refs=[], cfg=False, desc="1024x1024: 4096 image + 512 text tokens"),
    "c5": dict(h=32, w=32, txt=512, refs=[(32, 32, 10)], cfg=True,
               desc="512x512 CFG + 1 reference image: 2 forwards/step over 2048 image + 512 text tokens"),
}


def load_model(cfg, seed=42, qk="literal"):
    m = fluxhip.Transformer(cfg)
    for name in tensor_shapes(cfg):
        m.set_tensor(name, make_weights(cfg, seed, 0.02, qk, only=[name])[name])
    return m


EPI_QKV_SWIGLU = 8          # flux_hip_linear_probe's number for the launches of flux_hip_linear_qkv_swiglu


def dominant_kernel_cost(cfg, tokens, fused):
    """Algorithmic FLOPs and bytes of one launch of the step's dominant kernel: the [Q|K|V|gate|up] projection of a
    single-stream block (fused) or the gate/up projection with SwiGLU epilogue (not fused), each operand read once
    and each output written once, bf16."""
    H, M = cfg.hidden, cfg.mlp
    if fused:
        return 2.0 * tokens * H * (3 * H + 2 * M), 2.0 * ((3 * H + 2 * M) * H + tokens * H + tokens * (3 * H + M))
    return 2.0 * tokens * H * 2 * M, 2.0 * (2 * M * H + tokens * H + tokens * M)


def time_dominant_kernel(cfg, tokens, fused, launches=20):
    """The dominant kernel alone, back to back on resident buffers, at [tokens, hidden]: ms per launch."""
    import ctypes
    H, M = cfg.hidden, cfg.mlp
    rows = 3 * H + 2 * M if fused else 2 * M
    a = fluxhip.DevBuf.from_array(normal_bf16((tokens, H), 5, 1))
    w = fluxhip.DevBuf.from_array(normal_bf16((rows, H), 5, 2, 0.0, 0.02))
    out = fluxhip.DevBuf(tokens * M * 2)
    qkv = fluxhip.DevBuf(tokens * 3 * H * 2) if fused else None
    L = fluxhip.lib()
    L.flux_hip_linear_qkv_swiglu.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 8

    def run():
        if fused:
            fluxhip.check(L.flux_hip_linear_qkv_swiglu(a.ptr, w.ptr, qkv.ptr, out.ptr, tokens, 3 * H, M, H, H, H, 3 * H, M), "flux_hip_linear_qkv_swiglu")
        else:
            fluxhip.linear(fluxhip.EPI_SWIGLU, [(a.ptr, w.ptr, out.ptr, None, tokens)], 2 * M, H, H, H, M, 0, M)

    for _ in range(5):
        run()
    fluxhip.sync()
    L.flux_hip_timer_start()
    for _ in range(launches):
        run()
    ms = L.flux_hip_timer_stop() / launches
    for b in (a, w, out, qkv):
        if b is not None:
            b.free()
    return ms


def cpu_baseline(cfg, wl, forwards):
    """The CPU oracle on this host: ONE whole forward of the workload (input projections, timestep MLP and
    modulation, all double- and single-stream blocks, final layer) at full shape, timed after a small warm-up
    forward that touches every weight -> steps/s (a CFG step is two such forwards)."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle as O
    blas = O.enable_blas()
    o = O.Oracle(cfg, {})
    for name in tensor_shapes(cfg):                      # one tensor at a time on the host (15.5 GB as fp32 in the oracle)
        a = make_weights(cfg, 42, 0.02, "literal", only=[name])[name]
        assert O.lib().fo_model_set_bf16(o.h, name.encode(), a.ctypes.data, a.size) == 0, name
    h, w, nt = wl["h"], wl["w"], wl["txt"]
    refs = [(normal_f32((cfg.channels, rh, rw), 123, 10 + i), rh, rw, t) for i, (rh, rw, t) in enumerate(wl["refs"])]
    o.forward(normal_f32((cfg.channels, 2, 2), 9, 1), 2, 2, normal_f32((8, cfg.text_dim), 9, 2), 1.0)   # warm-up: 12 tokens
    z = normal_f32((cfg.channels, h, w), 123, 1)
    txt = normal_f32((nt, cfg.text_dim), 123, 2)
    t0 = time.time()
    v = o.forward(z, h, w, txt, 1.0, refs=refs)
    t_fwd = time.time() - t0
    assert np.isfinite(v).all()
    o.close()
    n = h * w + sum(rh * rw for rh, rw, _ in wl["refs"]) + nt
    threads = int(O.lib().fo_num_threads())
    return {
        "value": 1.0 / (forwards * t_fwd), "unit": "steps/s", "cores": threads, "kind": "port",
        "sample": f"1 full forward of the CPU oracle ({t_fwd:.2f} s: embedders, {cfg.n_double} double- and {cfg.n_single} single-stream "
                  f"blocks, final layer; {n} tokens) after a 12-token warm-up forward"
                  + (f", times {forwards} forwards per step" if forwards > 1 else "") + "; "
                  + (f"GEMMs: OpenBLAS sgemm ({os.path.basename(blas)}) on {threads} threads" if blas else f"GEMMs: built-in OpenMP loops on {threads} threads")
                  + f", os.cpu_count() = {os.cpu_count()}; the oracle's other loops (AdaLN, QK-norm, RoPE, softmax, SiLU) are OpenMP-parallel "
                    "on the same threads, where the reference runs them on one thread (flux_transformer.c:1021-1046), so this "
                    "baseline is at least as fast as the reference's BLAS build would be on this host",
    }


VAE_WORKLOADS = {"vae_c2": 16, "vae_c3": 32, "vae_c4": 64,   # latent side: 256^2, 512^2, 1024^2 images
                 "vae_enc_c2": 16, "vae_enc_c3": 32, "vae_enc_c4": 64}   # the same sizes through the encoder


def vae_cpu_baseline(flops_step, encode=False):
    """The CPU oracle's decoder / encoder (OpenMP loops) on a 128x128 (256x256) image; its FLOP rate
    carried to the benchmarked size."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle as O
    from model_spec import make_vae_weights, vae_decode_flops, vae_encode_flops, vae_test_image
    o = O.VaeOracle(make_vae_weights())
    if encode:
        o.encode(vae_test_image(32, 32, 9))
        img = vae_test_image(256, 256, 9)
        t0 = time.perf_counter()
        o.encode(img)
        dt = time.perf_counter() - t0
        rate, what, unit = vae_encode_flops(256, 256) / dt, "256x256 encode", "encodes/s"
    else:
        lat = normal_f32((128, 8, 8), 9, 1)
        o.decode(normal_f32((128, 2, 2), 9, 2), 2, 2)
        t0 = time.perf_counter()
        o.decode(lat, 8, 8)
        dt = time.perf_counter() - t0
        rate, what, unit = vae_decode_flops(8, 8) / dt, "128x128 decode", "decodes/s"
    o.close()
    return {"value": rate / flops_step, "unit": unit, "cores": O.lib().fo_num_threads(), "kind": "port",
            "sample": f"one {what} ({dt:.1f} s, {rate / 1e9:.1f} GFLOP/s, OpenMP loops of the CPU oracle), "
                      f"carried to this size by FLOP count"}


def bench_vae(args):
    """One step = one decode of a latent to an 8-bit image through flux_hip_vae_decode (host latent in,
    host image out: 0.5 + 3 MB over PCIe at 1024^2, inside the timed region), or (vae_enc_*) one encode
    of an fp32 image to a latent through flux_hip_vae_encode (12.6 + 0.5 MB over PCIe at 1024^2)."""
    import ctypes
    from model_spec import make_vae_weights, vae_decode_convs, vae_decode_flops, vae_encode_convs, vae_encode_flops, vae_test_image
    side = VAE_WORKLOADS[args.workload]
    enc = args.workload.startswith("vae_enc")
    K, Wm = args.steps, args.warmup
    fluxhip.init()
    if args.tile_mask:
        fluxhip.lib().flux_hip_linear_tile_mask(args.tile_mask)
    v = fluxhip.Vae(make_vae_weights())
    if enc:
        img = vae_test_image(16 * side, 16 * side, 322)
        step = lambda: v.encode(img)
        for _ in range(max(Wm, 1)):
            z = step()
        assert np.isfinite(z).all() and z.std() > 0.2
    else:
        lat = normal_f32((128, side, side), 321, 1)
        step = lambda: v.decode(lat, side, side)
        for _ in range(max(Wm, 1)):
            f, u = step()
        assert np.isfinite(f).all() and u.std() > 5.0
    L = fluxhip.lib()
    if not args.no_kernel_timing:
        L.flux_hip_linear_probe(-2)          # events around every convolution launch
    t0 = time.perf_counter()
    for _ in range(K):
        step()
    wall = time.perf_counter() - t0
    flops = vae_encode_flops(16 * side, 16 * side) if enc else vae_decode_flops(side, side)
    roof = None
    if not args.no_kernel_timing:
        # launch i of a decode is convolution i of vae_decode_convs (after the post-quant one, which the
        # input kernel does); a kernel (= tile shape) runs layers of several shapes, so its figure is
        # (sum of its launches' algorithmic FLOPs) / (sum of their durations). Dominant = most time.
        convs = vae_encode_convs(16 * side, 16 * side) if enc else vae_decode_convs(side, side)[1:]
        cap = K * len(convs)
        tiles = np.zeros(cap, np.int32)
        ms = np.zeros(cap, np.float32)
        n = L.flux_hip_linear_probe_read_launches(cap, tiles.ctypes.data, ms.ctypes.data)
        L.flux_hip_linear_probe(-1)
        if n == cap:
            fl = np.array([2.0 * H * W * ci * co * t for _, H, W, ci, co, t in convs] * K)
            names = {0: "gemm_kernel<64,128,2,2,CONV>", 1: "gemm_kernel<128,128,2,2,CONV>", 2: "gemm4w_kernel<8,8,CONV> (256x256 tile)",
                     3: "gemm_kernel<64,64,2,2,CONV>"}
            per_tile = {int(t): (float(ms[tiles == t].sum()), float(fl[tiles == t].sum()), int((tiles == t).sum())) for t in np.unique(tiles)}
            dom = max(per_tile, key=lambda t: per_tile[t][0])
            t_ms, t_fl, t_n = per_tile[dom]
            ach = t_fl / (t_ms * 1e-3) / 1e12
            roof = {"bound": "mfma", "achieved": round(ach, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(ach / PEAK_BF16_TFLOPS, 4), "traffic": None,
                    "kernel": names.get(dom, f"tile {dom}") + ": 3x3 / 1x1 convolutions as GEMMs with bias, residual and border epilogue",
                    "launches_timed": t_n, "ms_per_launch": round(t_ms / t_n, 4), "flops_per_launch": t_fl / t_n,
                    "launches_per_step": t_n // K,
                    "all_conv_kernels": {names.get(t, str(t)): {"launches_per_step": c // K, "ms_per_step": round(m / K, 3),
                                                                "tflops": round(f / (m * 1e-3) / 1e12, 1)} for t, (m, f, c) in per_tile.items()}}
    v.close()
    cpu = None if args.no_cpu_baseline else vae_cpu_baseline(flops, enc)
    what = "encodes" if enc else "decodes"
    print(json.dumps({
        "metric": f"VAE {what}/s ({16 * side}x{16 * side} image, 1 GPU)", "value": round(K / wall, 3), "unit": f"{what}/s",
        "n_gpus": 1, "steps": K, "warmup": Wm, "ms_per_step": round(wall * 1000.0 / K, 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": (f"{args.workload}: FLUX.2 VAE encoder (random-init bf16), {16 * side}x{16 * side} RGB fp32 -> latent "
                                f"[128,{side},{side}], batch 1, host buffers in and out") if enc else
                               (f"{args.workload}: FLUX.2 VAE decoder (84 M parameters, random-init bf16), latent "
                                f"[128,{side},{side}] -> {16 * side}x{16 * side} RGB, batch 1, host buffers in and out")},
        "tflops": round(flops * K / wall / 1e12, 1), "flops_per_step": flops, "roofline": roof, "cpu_baseline": cpu}))


def bench_qwen3(args):
    """One step = one text-encoder forward over 512 tokens (the padded length the pipeline always uses,
    flux_qwen3.c:1627-1652) through flux_hip_qwen3_forward: host token ids in, host embeddings
    [512, 7680] fp32 out (15.7 MB over PCIe inside the timed region)."""
    import ctypes
    from model_spec import QWEN3_4B, qwen3_tensor_shapes, make_qwen3_weights, qwen3_flops
    cfg = QWEN3_4B
    K, Wm = args.steps, args.warmup
    seq, real = 512, 40
    fluxhip.init()
    if args.tile_mask:
        fluxhip.lib().flux_hip_linear_tile_mask(args.tile_mask)
    m = fluxhip.Qwen3(cfg)
    last = max(cfg.out_layers)
    for name in qwen3_tensor_shapes(cfg):
        if name.startswith("model.layers.") and int(name.split(".")[2]) > last:
            continue
        m.set_tensor(name, make_qwen3_weights(cfg, only=[name])[name])
    rng = np.random.default_rng(5)
    ids = rng.integers(0, cfg.vocab, seq).astype(np.int32)
    mask = np.zeros(seq, np.int32)
    mask[:real] = 1
    ids[real:] = 151643
    for _ in range(max(Wm, 1)):
        out = m.forward(ids, mask)
    assert np.isfinite(out).all()
    L = fluxhip.lib()
    if not args.no_kernel_timing:
        L.flux_hip_linear_probe(fluxhip.EPI_SWIGLU)
    t0 = time.perf_counter()
    for _ in range(K):
        m.forward(ids, mask)
    wall = time.perf_counter() - t0
    flops = qwen3_flops(cfg, seq)
    roof = None
    if not args.no_kernel_timing:
        n_t, ms_t = ctypes.c_int(0), ctypes.c_float(0.0)
        L.flux_hip_linear_probe_read(ctypes.byref(n_t), ctypes.byref(ms_t))
        L.flux_hip_linear_probe(-1)
        if n_t.value:
            k_flops = 2.0 * seq * cfg.hidden * 2 * cfg.intermediate
            per_ms = ms_t.value / n_t.value
            ach = k_flops / (per_ms * 1e-3) / 1e12
            roof = {"bound": "mfma", "achieved": round(ach, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(ach / PEAK_BF16_TFLOPS, 4), "traffic": None,
                    "kernel": "gate/up projection + SiLU*up GEMM at [512, 2560] x [19456, 2560]^T (the largest of a layer's four GEMMs)",
                    "launches_timed": n_t.value, "ms_per_launch": round(per_ms, 4), "flops_per_launch": k_flops}
    m.close()
    cpu = None
    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import oracle as O
        from dataclasses import replace
        # two full-size layers over 64 tokens on the CPU oracle, carried to the benchmarked size by FLOP count
        c2 = replace(cfg, layers=2, out_layers=(0, 1, 1), vocab=1024)
        o = O.Qwen3Oracle(c2, make_qwen3_weights(c2))
        ids_c = rng.integers(0, 1024, 64).astype(np.int32)
        o.forward(ids_c[:4])
        t1 = time.perf_counter()
        o.forward(ids_c)
        dt = time.perf_counter() - t1
        o.close()
        rate = qwen3_flops(c2, 64) / dt
        cpu = {"value": rate / flops, "unit": "encodes/s", "cores": O.lib().fo_num_threads(), "kind": "port",
               "sample": f"two full-size layers over 64 tokens ({dt:.1f} s, {rate / 1e9:.1f} GFLOP/s, OpenMP loops of the CPU oracle), "
                         f"carried to 27 layers x 512 tokens by FLOP count"}
    print(json.dumps({
        "metric": "text encodes/s (Qwen3-4B encoder, 512 tokens, 1 GPU)", "value": round(K / wall, 3), "unit": "encodes/s",
        "n_gpus": 1, "steps": K, "warmup": Wm, "ms_per_step": round(wall * 1000.0 / K, 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "qwen3: Qwen3-4B text encoder (layers 0-26 of 36, random-init bf16), 512 token ids "
                               "(40 real + padding) -> [512, 7680] embeddings, host buffers in and out"},
        "tflops": round(flops * K / wall / 1e12, 1), "flops_per_step": flops, "roofline": roof, "cpu_baseline": cpu}))


ATT_WORKLOADS = {"att_c1": 80, "att_c2": 768, "att_c3": 1536, "att_c4": 4608, "att_c5": 2560}   # tokens (text first: 64 at c1, else 512)


def bench_attention(args):
    """The attention operator alone at a workload's sequence length (24 heads of 128, text split at 512): one "step"
    is one flux_hip_qk_prepare + flux_hip_attention pair, back to back on resident buffers, as a single-stream
    block runs them. The roofline object is the attention kernel by itself (HIP events around runs of it)."""
    n, heads = ATT_WORKLOADS[args.workload], KLEIN_4B.heads
    H = heads * 128
    split = 64 if n < 512 else 512
    fluxhip.init()
    L = fluxhip.lib()
    L.flux_hip_attention_force_variant(args.attention_variant)
    qkv = fluxhip.DevBuf.from_array(normal_bf16((n, 3 * H), 5, 1))
    w = fluxhip.DevBuf.from_array(np.ones(128, np.float32))
    ang = normal_f32((n, 128), 5, 2)
    cos, sin = fluxhip.DevBuf.from_array(np.cos(ang)), fluxhip.DevBuf.from_array(np.sin(ang))
    kn, out = fluxhip.DevBuf(n * H * 2), fluxhip.DevBuf(n * H * 2)

    def prep():
        # Q is prepared in place: every pass normalises the Q columns again (finite, and the timing does not depend on the values)
        fluxhip.check(L.flux_hip_qk_prepare(kn.ptr, qkv.ptr, 3 * H, 0, H, n, heads, split, w.ptr, w.ptr, w.ptr, w.ptr, cos.ptr, sin.ptr, 1e-6))

    def att():
        fluxhip.check(L.flux_hip_attention(out.ptr, H, qkv.ptr, 3 * H, kn.ptr, qkv.at(2 * H * 2), 3 * H, n, n, heads))

    for _ in range(max(args.warmup, 1)):
        prep(); att()
    fluxhip.sync()
    t0 = time.perf_counter()
    L.flux_hip_timer_start()
    for _ in range(args.steps):
        prep(); att()
    ev_ms = L.flux_hip_timer_stop()
    wall = time.perf_counter() - t0
    L.flux_hip_timer_start()
    for _ in range(args.steps):
        att()
    att_ms = L.flux_hip_timer_stop() / args.steps
    L.flux_hip_timer_start()
    for _ in range(args.steps):
        prep()
    prep_ms = L.flux_hip_timer_stop() / args.steps
    res = bf16_to_f32_host(out.to_array(np.uint16, (n, H)))
    assert np.isfinite(res).all()
    flops = 4.0 * n * n * H
    ach = flops / (att_ms * 1e-3) / 1e12
    prep_bytes = 4.0 * n * H * 2
    L.flux_hip_attention_force_variant(-1)
    print(json.dumps({
        "metric": f"attention calls/s ({n} tokens, {heads} heads, 1 GPU)", "value": round(args.steps / wall, 2), "unit": "calls/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall * 1000.0 / args.steps, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: Q/K preparation + joint attention over {n} tokens ({split} text), {heads} heads x 128, N(0,1) bf16 "
                               f"q/k/v, unit QK-norm weights, random RoPE angles; variant {args.attention_variant}"},
        "device_ms_per_step_events": round(ev_ms / args.steps, 4),
        "roofline": {"bound": "mfma", "achieved": round(ach, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(ach / PEAK_BF16_TFLOPS, 4),
                     "traffic": None, "kernel": "attention_wide_kernel: softmax(q k^T / sqrt(128)) v, 4 n^2 H FLOP",
                     "ms_per_launch": round(att_ms, 4), "flops_per_launch": flops},
        "qk_prepare": {"bound": "hbm", "ms_per_launch": round(prep_ms, 4), "bytes_per_launch": prep_bytes,
                       "achieved_GBps": round(prep_bytes / (prep_ms * 1e-3) / 1e9, 1), "peak_GBps": 8000.0,
                       "frac": round(prep_bytes / (prep_ms * 1e-3) / 8e12, 4)},
        "cpu_baseline": None}))


BW_WORKLOADS = {"bw_c3": 1536, "bw_c4": 4608}


def bench_bandwidth(args):
    """The bandwidth-bound kernels of a block at a workload's token count, each alone on resident buffers: LayerNorm +
    modulation (flux_hip_adaln_norm: fp32 [tokens, 3072] in, bf16 out), Q/K preparation (flux_hip_qk_prepare: Q and K
    of 24 heads in, normalised + rotated Q (in place) and K out) and, as the yardstick for what a trivial streaming
    kernel reaches at this size, the fp32 -> bf16 conversion over the same element count. Every kernel is timed twice:
    launches over the same buffers (operands stay in the 256 MB memory-side cache) and over four buffer sets in turn
    (every launch finds its operands in HBM). One "step" is one launch of each kernel on rotating buffers."""
    n, heads, H = BW_WORKLOADS[args.workload], KLEIN_4B.heads, KLEIN_4B.hidden
    fluxhip.init()
    L = fluxhip.lib()
    NB = 4
    launches = max(args.steps, 1)

    def timed(fn):
        for i in range(max(args.warmup, 1) * NB):
            fn(i)
        fluxhip.sync()
        L.flux_hip_timer_start()
        for i in range(launches):
            fn(i)
        return L.flux_hip_timer_stop() / launches

    x = [fluxhip.DevBuf.from_array(normal_f32((n, H), 7, i)) for i in range(NB)]
    o = [fluxhip.DevBuf(n * H * 2) for _ in range(NB)]
    sh, sc = fluxhip.DevBuf.from_array(normal_f32((H,), 7, 20)), fluxhip.DevBuf.from_array(normal_f32((H,), 7, 21))
    qkv = [fluxhip.DevBuf.from_array(normal_bf16((n, 3 * H), 5, i)) for i in range(NB)]
    w = fluxhip.DevBuf.from_array(np.ones(128, np.float32))
    ang = normal_f32((n, 128), 5, 2)
    cos, sin = fluxhip.DevBuf.from_array(np.cos(ang)), fluxhip.DevBuf.from_array(np.sin(ang))
    kn = [fluxhip.DevBuf(n * H * 2) for _ in range(NB)]

    def adaln(j):
        fluxhip.check(L.flux_hip_adaln_norm(o[j].ptr, H, x[j].ptr, n, H, 512, sh.ptr, sc.ptr, sh.ptr, sc.ptr, 1e-6))

    def prep(j):
        fluxhip.check(L.flux_hip_qk_prepare(kn[j].ptr, qkv[j].ptr, 3 * H, 0, H, n, heads, 512, w.ptr, w.ptr, w.ptr, w.ptr, cos.ptr, sin.ptr, 1e-6))

    def conv(j):
        fluxhip.check(L.flux_hip_f32_to_bf16(o[j].ptr, x[j].ptr, n * H))

    kernels = {"adaln_kernel": (adaln, 6.0 * n * H, "fp32 row in, bf16 row out: 6 bytes per element"),
               "qk_prepare_kernel": (prep, 8.0 * n * H, "bf16 Q and K in, bf16 Q and K out: 8 bytes per element of K (the cos/sin rows, 1 KB per token, "
                                                            "which every head reads again from L2, not counted)"),
               "f32_to_bf16_kernel": (conv, 6.0 * n * H, "yardstick: same bytes as adaln_kernel, no reduction")}
    table = {}
    t0 = time.perf_counter()
    for name, (fn, nbytes, what) in kernels.items():
        warm = timed(lambda i: fn(0))
        cold = timed(lambda i: fn(i % NB))
        table[name] = {"bytes_per_launch": nbytes, "what": what,
                       "same_buffers": {"us": round(warm * 1e3, 2), "GBps": round(nbytes / warm / 1e6, 1), "frac_of_hbm_peak": round(nbytes / warm / 1e6 / PEAK_HBM_GBPS, 4)},
                       "four_buffer_sets_in_turn": {"us": round(cold * 1e3, 2), "GBps": round(nbytes / cold / 1e6, 1),
                                                    "frac_of_hbm_peak": round(nbytes / cold / 1e6 / PEAK_HBM_GBPS, 4)}}
    wall = time.perf_counter() - t0
    a = table["adaln_kernel"]["four_buffer_sets_in_turn"]
    print(json.dumps({
        "metric": f"launches/s of the bandwidth-bound kernels ({n} tokens, 1 GPU)", "value": round(6 * launches / wall, 1), "unit": "launches/s",
        "n_gpus": 1, "steps": launches, "warmup": args.warmup, "ms_per_step": None, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}: adaln_kernel, qk_prepare_kernel and the fp32->bf16 yardstick at [{n}, {H}], N(0,1) inputs"},
        "roofline": {"bound": "hbm", "achieved": a["GBps"], "peak": PEAK_HBM_GBPS, "unit": "GB/s", "frac": a["frac_of_hbm_peak"], "traffic": None,
                     "kernel": "adaln_kernel, operands in HBM (four buffer sets in turn)"},
        "kernels": table, "cpu_baseline": None}))


GEMM_SHAPES = {"qkv": (4608, 9216, 3072), "gate_up": (4608, 18432, 3072), "fused_qkv_gate_up": (4608, 27648, 3072),
               "out_k12288": (4608, 3072, 12288)}


def bench_gemm_vs_library(args):
    """The step's four big projection shapes as plain bf16 GEMMs C = A W^T (bf16 store, no fused epilogue), this
    backend's flux_hip_linear against the vendor library behind torch.matmul (hipBLASLt / rocBLAS), each back to
    back on resident N(0,1) x N(0,0.02) operands: once over the same buffers (operands stay in the memory-side cache)
    and once over four buffer sets in turn (operands come from HBM, as the weights of every layer do in a step)."""
    import torch
    fluxhip.init()
    L = fluxhip.lib()
    L.flux_hip_linear_enable_splitk(0)
    NB, launches, warm = 4, max(args.steps, 4), 40
    rows = {}
    t0 = time.perf_counter()
    for name, (M, N, K) in GEMM_SHAPES.items():
        a_h = [normal_bf16((M, K), 5, 10 + i) for i in range(NB)]
        w_h = [normal_bf16((N, K), 5, 20 + i, 0.0, 0.02) for i in range(NB)]
        a = [fluxhip.DevBuf.from_array(x) for x in a_h]
        w = [fluxhip.DevBuf.from_array(x) for x in w_h]
        c = fluxhip.DevBuf(M * N * 2)

        def mine(j):
            fluxhip.linear(fluxhip.EPI_BF16, [(a[j].ptr, w[j].ptr, c.ptr, None, M)], N, K, K, K, N)

        ta = [torch.from_numpy(x.view(np.int16)).cuda().view(torch.bfloat16) for x in a_h]
        tw = [torch.from_numpy(x.view(np.int16)).cuda().view(torch.bfloat16) for x in w_h]
        out = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")

        def lib(j):
            torch.matmul(ta[j], tw[j].t(), out=out)

        def timed_mine(rot):
            for i in range(warm):
                mine(i % NB if rot else 0)
            fluxhip.sync()
            L.flux_hip_timer_start()
            for i in range(launches):
                mine(i % NB if rot else 0)
            return L.flux_hip_timer_stop() / launches

        def timed_lib(rot):
            for i in range(warm):
                lib(i % NB if rot else 0)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(launches):
                lib(i % NB if rot else 0)
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / launches

        # the clocks take a second to settle after the uploads, and they drift with what ran before: the four
        # measurements take turns, three rounds, and each reports its best round
        m_same = m_rot = l_same = l_rot = 1e9
        for _ in range(3):
            m_same = min(m_same, timed_mine(False))
            l_same = min(l_same, timed_lib(False))
            m_rot = min(m_rot, timed_mine(True))
            l_rot = min(l_rot, timed_lib(True))
        mine(0)
        fluxhip.sync()
        got = bf16_to_f32_host(c.to_array(np.uint16, (M, N))[:64])
        lib(0)
        ref = out[:64].float().cpu().numpy()
        err = float(np.linalg.norm(got - ref) / np.linalg.norm(ref))
        assert err < 1e-2, (name, err)
        fl = 2.0 * M * N * K
        rows[name] = {"M": M, "N": N, "K": K, "gflop": round(fl / 1e9, 1),
                      "flux_hip_linear": {"same_buffers_us": round(m_same * 1e3, 1), "rotating_us": round(m_rot * 1e3, 1),
                                          "same_buffers_tflops": round(fl / m_same / 1e9, 1), "rotating_tflops": round(fl / m_rot / 1e9, 1)},
                      "library": {"same_buffers_us": round(l_same * 1e3, 1), "rotating_us": round(l_rot * 1e3, 1),
                                  "same_buffers_tflops": round(fl / l_same / 1e9, 1), "rotating_tflops": round(fl / l_rot / 1e9, 1)},
                      "rel_l2_between_the_two": round(err, 5)}
        for b in a + w + [c]:
            b.free()
        del ta, tw, out
        torch.cuda.empty_cache()
    wall = time.perf_counter() - t0
    worst = min(r["flux_hip_linear"]["rotating_tflops"] / r["library"]["rotating_tflops"] for r in rows.values())
    k = rows["fused_qkv_gate_up"]["flux_hip_linear"]
    print(json.dumps({
        "metric": "bf16 GEMM TFLOP/s on the step's projection shapes, this backend against the vendor library (1 GPU)",
        "value": k["rotating_tflops"], "unit": "TFLOP/s", "n_gpus": 1, "steps": launches, "warmup": warm, "ms_per_step": None,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "gemm_vs_lib: C = A W^T, bf16 in and out, fp32 accumulation; value = flux_hip_linear at [4608,3072] x [27648,3072]^T "
                               f"with operands from HBM; library = torch {torch.__version__} matmul"},
        "worst_ratio_to_library_rotating": round(worst, 3), "shapes": rows, "wall_s": round(wall, 1),
        "roofline": {"bound": "mfma", "achieved": k["rotating_tflops"], "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(k["rotating_tflops"] / PEAK_BF16_TFLOPS, 4), "traffic": None,
                     "kernel": "gemm4d_kernel, bf16 store, back to back, four buffer sets in turn"},
        "cpu_baseline": None}))


def bench_mfma_issue(args):
    """What another instruction costs a lone wave when it sits between that wave's MFMAs (flux_hip_mfma_issue_cost:
    one workgroup of four waves per compute unit, 16 independent accumulator blocks per wave, one instruction of the
    given kind behind every n-th MFMA): clock cycles per MFMA, 16 = the matrix pipe never waits. The GEMM and
    attention kernels run one wave per SIMD, so these are the costs their loops pay."""
    import ctypes
    fluxhip.init()
    L = fluxhip.lib()
    L.flux_hip_mfma_issue_cost.argtypes = [ctypes.c_int] * 3 + [ctypes.POINTER(ctypes.c_float)] * 2
    kinds = {0: "nothing", 1: "global_load_lds_dwordx4", 2: "ds_read_b128", 3: "v_exp_f32", 4: "3 x v_fma_f32",
             5: "global_load_dwordx4 + ds_write_b128"}
    iters = 4000
    table = []
    for mode, name in kinds.items():
        for every in ((4,) if mode == 0 else (16, 8, 4, 2, 1)):
            c, g = ctypes.c_float(0.0), ctypes.c_float(0.0)
            fluxhip.check(L.flux_hip_mfma_issue_cost(mode, every, iters, ctypes.byref(c), ctypes.byref(g)), "flux_hip_mfma_issue_cost")
            table.append({"between_the_mfmas": name, "one_per_mfmas": every, "cycles_per_mfma": round(c.value, 2), "core_ghz": round(g.value, 2)})
    base = table[0]["cycles_per_mfma"]
    for r in table[1:]:
        r["cycles_per_instruction_beyond_the_loop_alone"] = round((r["cycles_per_mfma"] - base) * r["one_per_mfmas"], 1)
    dma8 = next(r for r in table if r["between_the_mfmas"] == "global_load_lds_dwordx4" and r["one_per_mfmas"] == 8)
    print(json.dumps({
        "metric": "matrix-pipe cycles per MFMA of a lone wave with one global->LDS load behind every 8th MFMA (16 = no loss, 1 GPU)",
        "value": dma8["cycles_per_mfma"], "unit": "cycles", "n_gpus": 1, "steps": 2, "warmup": 1, "ms_per_step": None,
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"mfma_issue: {iters} x 16 v_mfma_f32_16x16x32_bf16 per wave, four waves per compute unit, one other instruction "
                               "behind every n-th MFMA"},
        "table": table, "roofline": None, "cpu_baseline": None}))


def bf16_to_f32_host(a):
    return (a.astype(np.uint32) << 16).view(np.float32)


def bench_mfma_peak(args):
    """The matrix pipes on their own (flux_hip_mfma_peak: register-resident loops of independent bf16 MFMAs on every
    compute unit, no memory traffic), for both instruction shapes, one and two waves per SIMD, and operand data of
    three kinds. One "step" is one launch of about 5 ms; the figure is the best of --steps launches after --warmup."""
    import ctypes
    fluxhip.init()
    L = fluxhip.lib()
    L.flux_hip_mfma_peak.argtypes = [ctypes.c_int] * 5 + [ctypes.POINTER(ctypes.c_float)]
    shapes = {0: "v_mfma_f32_16x16x32_bf16", 1: "v_mfma_f32_32x32x16_bf16"}
    patterns = {0: "all zeros", 1: "1.0 <= x < 2.0, random low byte", 2: "random bit patterns"}
    iters = 12000                       # x 16 MFMAs per wave: about 5 ms per launch at two waves per SIMD
    table = []
    for waves in (2, 1):
        for pat in patterns:
            row = {"operands": patterns[pat], "waves_per_simd": waves}
            for sh in shapes:
                t = ctypes.c_float(0.0)
                for _ in range(max(args.warmup, 0)):
                    fluxhip.check(L.flux_hip_mfma_peak(sh, pat, waves, iters, 1, ctypes.byref(t)), "flux_hip_mfma_peak")
                fluxhip.check(L.flux_hip_mfma_peak(sh, pat, waves, iters, max(args.steps, 1), ctypes.byref(t)), "flux_hip_mfma_peak")
                row[shapes[sh]] = round(t.value, 1)
            table.append(row)
    best = max(r[shapes[0]] for r in table if r["operands"] == "random bit patterns")
    zeros = max(max(r[shapes[0]], r[shapes[1]]) for r in table if r["operands"] == "all zeros")
    print(json.dumps({
        "metric": "MFMA-only bf16 throughput, operands in registers (TFLOP/s, 1 GPU)", "value": best, "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": None, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "mfma_peak: one workgroup per compute unit, 16 independent accumulator blocks (64 registers) per wave, "
                               f"{iters} x 16 MFMAs per wave and launch; value = v_mfma_f32_16x16x32_bf16 on random bit patterns"},
        "datasheet_peak": PEAK_BF16_TFLOPS, "best_on_zero_operands": zeros, "frac_of_datasheet_on_random_bits": round(best / PEAK_BF16_TFLOPS, 4),
        "table": table, "roofline": None, "cpu_baseline": None}))


def measure_workload(model, cfg, name, K, Wm, fused, args, headline):
    """Wm untimed + K timed denoising steps of workload `name` through the session API on the resident model: inputs,
    text and every step's modulation are in HBM before the timed region, which is bracketed by stream synchronisation
    (wall clock) and by HIP events on the backend's stream; HIP events around every launch of the dominant kernel."""
    import ctypes
    wl = WORKLOADS[name]
    h, w, nt = wl["h"], wl["w"], wl["txt"]
    n_target = h * w
    n_img = n_target + sum(rh * rw for rh, rw, _ in wl["refs"])
    forwards = 2 if wl["cfg"] else 1
    z = normal_f32((cfg.channels, h, w), 123, 1)
    txt = normal_f32((nt, cfg.text_dim), 123, 2)
    txt_u = normal_f32((nt, cfg.text_dim), 123, 3) if wl["cfg"] else None
    refs = [(normal_f32((cfg.channels, rh, rw), 123, 10 + i), rh, rw, t) for i, (rh, rw, t) in enumerate(wl["refs"])]
    sched = fluxhip.schedule("official", K + Wm, n_target)
    sess = fluxhip.Session(model, z, h, w, txt, sched, refs=refs, txt_uncond=txt_u, guidance=4.0)

    for i in range(Wm):
        sess.step(i)
    sess.latent()                            # (reading the latent also collects the stage events recorded so far)
    fluxhip.sync()
    stages_warm = fluxhip.stage_timing()     # the stage counters run from the session's first step on: the timed steps' share is the difference
    L = fluxhip.lib()
    if not args.no_kernel_timing:
        L.flux_hip_linear_probe(EPI_QKV_SWIGLU if fused else fluxhip.EPI_SWIGLU)   # events around the dominant kernel's launches
    t0 = time.perf_counter()
    L.flux_hip_timer_start()
    for i in range(Wm, Wm + K):
        sess.step(i)
    ev_ms = L.flux_hip_timer_stop()      # waits for the last kernel
    fluxhip.sync()
    wall = time.perf_counter() - t0
    k_n, k_ms = ctypes.c_int(0), ctypes.c_float(0.0)
    # one projection runs under more than one tile shape in a step when it is launched at several sizes (the
    # two-part launches of the double-stream blocks); the dominant kernel is the shape with the most time
    epi_name = "QKV_SWIGLU" if fused else "SWIGLU"
    TILE_NAMES = {0: f"gemm_kernel<64,128,2,2,{epi_name}>", 1: f"gemm_kernel<128,128,2,2,{epi_name}>", 2: f"gemm4d_kernel<8,8,{epi_name}> (256x256 tile)",
                  3: f"gemm_kernel<64,64,2,2,{epi_name}>", 4: f"gemm_kernel<256,256,2,4,{epi_name}>", 5: f"gemm4d_kernel<9,6,{epi_name}> (288x192 tile)",
                  6: f"gemm4d_kernel<6,6,{epi_name}> (192x192 tile)", 7: f"gemm4d_kernel<8,6,{epi_name}> (256x192 tile)",
                  8: f"gemm_kernel<64,128,2,2,{epi_name},6> (ring of 6 stages)", 9: f"gemm_kernel<128,128,2,2,{epi_name},5> (ring of 5 stages)",
                  10: f"gemm_kernel<96,128,2,2,{epi_name},5> (ring of 5 stages)"}
    k_tile = -1
    for tile in TILE_NAMES:
        n_t, ms_t = ctypes.c_int(0), ctypes.c_float(0.0)
        L.flux_hip_linear_probe_read_tile(tile, ctypes.byref(n_t), ctypes.byref(ms_t))
        if ms_t.value > k_ms.value:
            k_tile, k_n, k_ms = tile, n_t, ms_t
    L.flux_hip_linear_probe(-1)
    zf = sess.latent()
    assert np.isfinite(zf).all(), "latent is not finite"
    stages = [a - b for a, b in zip(fluxhip.stage_timing(), stages_warm)]
    sess.close()

    # The drop-in sampler entry point on host buffers (upload of latent and text, modulation for
    # the schedule, 4 steps, download): the PCIe-inclusive figure, reported beside `value`, never as it.
    n_run, host_run_ms = 4, None
    if headline:
        s4 = fluxhip.schedule("official", n_run, n_target)
        model.sample(z, h, w, txt, s4, refs=refs, txt_uncond=txt_u, guidance=4.0)
        t1 = time.perf_counter()
        model.sample(z, h, w, txt, s4, refs=refs, txt_uncond=txt_u, guidance=4.0)
        host_run_ms = (time.perf_counter() - t1) * 1000.0

    ms_per_step = wall * 1000.0 / K
    flops_step = forwards * flops_per_forward(cfg, n_img, nt, n_target)
    tflops = flops_step / (wall / K) / 1e12

    roof = None
    if not args.no_kernel_timing and k_n.value > 0:
        # fused: only the single-stream blocks launch this kernel, all at [image + text tokens, H]; not fused: every
        # gate/up launch of the step, which all have that cost too
        per_ms = k_ms.value / k_n.value
        # a CFG step runs its two sequences as one batch: the launch then covers the rows of both
        seqs = forwards if (fused and not args.sequential_cfg) else 1
        k_flops, k_bytes = dominant_kernel_cost(cfg, seqs * (n_img + nt), fused)
        ach = k_flops / (per_ms * 1e-3) / 1e12
        gbps = k_bytes / (per_ms * 1e-3) / 1e9
        what = "[Q|K|V|gate|up] projection of a single-stream block, bf16 store + SiLU(gate)*up" if fused else "gate/up projection + SiLU*up"
        # the launch is bound by whichever of the two it needs longer for at the datasheet rates
        if k_flops / (PEAK_BF16_TFLOPS * 1e12) >= k_bytes / (PEAK_HBM_GBPS * 1e9):
            roof = {"bound": "mfma", "achieved": round(ach, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(ach / PEAK_BF16_TFLOPS, 4), "traffic": TRAFFIC_BYTES.get((name, fused))}
        else:
            roof = {"bound": "hbm", "achieved": round(gbps, 1), "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                    "frac": round(gbps / PEAK_HBM_GBPS, 4), "traffic": TRAFFIC_BYTES.get((name, fused))}
        roof.update({"kernel": TILE_NAMES[k_tile] + ": " + what, "launches_timed": k_n.value, "ms_per_launch": round(per_ms, 4),
                     "flops_per_launch": k_flops, "bytes_per_launch": k_bytes, "tflops": round(ach, 1), "GBps": round(gbps, 1)})
        if headline:
            roof["ms_per_launch_back_to_back"] = round(time_dominant_kernel(cfg, seqs * (n_img + nt), fused), 4)
    return {"ms_per_step": ms_per_step, "tflops": tflops, "flops_per_step": flops_step, "forwards": forwards, "roofline": roof,
            "stages": [x / K for x in stages], "ev_ms": ev_ms, "host_run_ms": host_run_ms, "host_run_steps": n_run, "steps": K,
            "tokens": n_img + nt}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=8)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="c4", choices=sorted(WORKLOADS) + sorted(VAE_WORKLOADS) + sorted(ATT_WORKLOADS) + sorted(BW_WORKLOADS) + ["qwen3", "mfma_peak", "mfma_issue", "gemm_vs_lib"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernel-timing", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="c4 only: leave out the short runs of c1, c2, c3 and c5 that follow the headline on the same weights")
    ap.add_argument("--tile-mask", type=lambda v: int(v, 0), default=0,
                    help="restrict the GEMM tiles the backend may choose (bit t = tile id t), for A/B runs")
    ap.add_argument("--sequential-cfg", action="store_true",
                    help="run the two forwards of a CFG step one after the other instead of as one batch (A/B runs)")
    ap.add_argument("--fused-qkv-mlp", type=int, default=1, choices=[0, 1],
                    help="single-stream blocks: 1 = QKV and gate/up projections as one launch (default), 0 = as two (A/B runs)")
    ap.add_argument("--ring", type=int, default=1, help="GEMM operand rings (flux_hip_linear_ring), for A/B runs")
    ap.add_argument("--attention-variant", type=int, default=-1,
                    help="attention kernel variant (flux_hip_attention_force_variant; -1 = the backend's choice), for A/B runs")
    ap.add_argument("--calibrate", action="store_true",
                    help="launch only a streaming kernel of known size (f32->bf16 over 64 Mi elements: reads 256 MiB, "
                         "writes 128 MiB) and the dominant GEMM, for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this backend runs the whole model on ONE GPU (no sharding, no collectives); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    if args.workload in VAE_WORKLOADS:
        return bench_vae(args)
    if args.workload == "qwen3":
        return bench_qwen3(args)
    if args.workload == "mfma_peak":
        return bench_mfma_peak(args)
    if args.workload in ATT_WORKLOADS:
        return bench_attention(args)
    if args.workload in BW_WORKLOADS:
        return bench_bandwidth(args)
    if args.workload == "gemm_vs_lib":
        return bench_gemm_vs_library(args)
    if args.workload == "mfma_issue":
        return bench_mfma_issue(args)
    cfg = KLEIN_4B
    wl = WORKLOADS[args.workload]
    if args.calibrate:
        fluxhip.init()
        n = 64 << 20
        src = fluxhip.DevBuf(n * 4)
        dst = fluxhip.DevBuf(n * 2)
        fluxhip.lib().flux_hip_memset(src.ptr, 0, n * 4)
        for _ in range(3):
            fluxhip.check(fluxhip.lib().flux_hip_f32_to_bf16(dst.ptr, src.ptr, n))
        fluxhip.sync()
        tokens = wl["h"] * wl["w"] + sum(rh * rw for rh, rw, _ in wl["refs"]) + wl["txt"]
        ms = time_dominant_kernel(cfg, tokens, bool(args.fused_qkv_mlp), launches=5)
        fl, by = dominant_kernel_cost(cfg, tokens, bool(args.fused_qkv_mlp))
        print(json.dumps({"calibration_copy": {"read_MiB": 256, "write_MiB": 128}, "gemm_ms": ms, "gemm_tflops": fl / ms / 1e9,
                          "gemm_algorithmic_bytes": by}))
        return
    K, Wm = args.steps, args.warmup
    fused = bool(args.fused_qkv_mlp)

    fluxhip.init()
    if args.tile_mask:
        fluxhip.lib().flux_hip_linear_tile_mask(args.tile_mask)
    if args.sequential_cfg:
        fluxhip.lib().flux_hip_set_batched_cfg(0)
    fluxhip.lib().flux_hip_set_fused_qkv_mlp(args.fused_qkv_mlp)
    fluxhip.lib().flux_hip_linear_ring(args.ring)
    fluxhip.lib().flux_hip_attention_force_variant(args.attention_variant)
    model = load_model(cfg)
    head = measure_workload(model, cfg, args.workload, K, Wm, fused, args, headline=True)
    ms_per_step, tflops, flops_step, forwards = head["ms_per_step"], head["tflops"], head["flops_per_step"], head["forwards"]
    roof, stages, ev_ms, host_run_ms, n_run = head["roofline"], head["stages"], head["ev_ms"], head["host_run_ms"], head["host_run_steps"]

    # The other configurations of the benchmark on the same resident weights, so that one line carries all five: a short
    # run each (same timing brackets, same probe on the dominant kernel), no CPU baseline of their own.
    others = None
    if args.workload == "c4" and not args.no_other_configs:
        others = {}
        for name in ("c1", "c2", "c3", "c5"):
            r = measure_workload(model, cfg, name, max(4, min(K, 8)), 2, fused, args, headline=False)
            others[name] = {"workload": WORKLOADS[name]["desc"], "ms_per_step": round(r["ms_per_step"], 3), "steps_per_s": round(1000.0 / r["ms_per_step"], 3),
                            "steps": r["steps"], "tflops": round(r["tflops"], 1), "frac_of_bf16_peak": round(r["tflops"] / PEAK_BF16_TFLOPS, 4),
                            "forwards_per_step": r["forwards"], "roofline": r["roofline"]}
    model.close()

    # What this box's matrix pipes sustain on their own (register-resident v_mfma_f32_16x16x32_bf16 on random bit patterns, two
    # waves per SIMD, best of three 5 ms launches): boxes differ by several per cent under the power limit, and the step follows.
    box = None
    if not args.no_kernel_timing:
        import ctypes
        Lb = fluxhip.lib()
        Lb.flux_hip_mfma_peak.argtypes = [ctypes.c_int] * 5 + [ctypes.POINTER(ctypes.c_float)]
        t = ctypes.c_float(0.0)
        fluxhip.check(Lb.flux_hip_mfma_peak(0, 2, 2, 12000, 1, ctypes.byref(t)), "flux_hip_mfma_peak")
        fluxhip.check(Lb.flux_hip_mfma_peak(0, 2, 2, 12000, 3, ctypes.byref(t)), "flux_hip_mfma_peak")
        box = {"mfma_only_tflops_random_bits": round(t.value, 1), "step_tflops_over_it": round(tflops / t.value, 4)}

    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(cfg, wl, forwards)

    out = {
        "metric": "transformer denoise steps/s at 1024^2 (1 GPU); achieved TFLOP/s vs bf16 peak"
                  if args.workload == "c4" else f"transformer denoise steps/s ({args.workload}, 1 GPU)",
        "value": round(1000.0 / ms_per_step, 4), "unit": "steps/s", "n_gpus": 1, "steps": K, "warmup": Wm,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: FLUX.2-klein-4B transformer, {wl['desc']}, batch 1, "
                               f"{forwards} forward(s)/step, random-init bf16 weights N(0,0.02)"},
        "tflops": round(tflops, 1), "frac_of_bf16_peak": round(tflops / PEAK_BF16_TFLOPS, 4),
        "flops_per_step": flops_step, "device_ms_per_step_events": round(ev_ms / K, 3),
        "host_buffer_run": {"steps": n_run, "ms": round(host_run_ms, 2),
                            "steps_per_s": round(n_run / host_run_ms * 1000.0, 3)},
        "stage_ms_per_step": {"double": round(stages[0], 3), "single": round(stages[1], 3), "final": round(stages[2], 3)},
        "roofline": roof, "cpu_baseline": cpu, "box": box, "other_configs": others,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
