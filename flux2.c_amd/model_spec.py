"""Architecture description and synthetic tensors for the FLUX.2-klein denoising transformer.

The tensor names and shapes are the safetensors keys the reference loader reads
(flux_transformer.c:4452-4602); the default sizes are flux.h:33-41.
"""
import ctypes
import os
from collections import OrderedDict
from dataclasses import dataclass, asdict

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))


@dataclass(frozen=True)
class FluxConfig:
    hidden: int = 3072
    heads: int = 24
    head_dim: int = 128
    mlp: int = 9216
    n_double: int = 5
    n_single: int = 20
    text_dim: int = 7680
    channels: int = 128
    axis_dim: int = 32
    sincos_dim: int = 256
    rope_theta: float = 2000.0

    def as_dict(self):
        return asdict(self)


KLEIN_4B = FluxConfig()
# A structurally identical model small enough for the CPU oracle to run in well under a second.
TINY = FluxConfig(hidden=256, heads=2, mlp=768, n_double=2, n_single=3, text_dim=384)
# One size up: 4 heads, used to exercise multi-tile GEMM/attention shapes.
SMALL = FluxConfig(hidden=512, heads=4, mlp=1536, n_double=2, n_single=4, text_dim=768)


def tensor_shapes(cfg: FluxConfig) -> "OrderedDict[str, tuple]":
    H, M, hd = cfg.hidden, cfg.mlp, cfg.head_dim
    t = OrderedDict()
    t["x_embedder.weight"] = (H, cfg.channels)
    t["context_embedder.weight"] = (H, cfg.text_dim)
    t["time_guidance_embed.timestep_embedder.linear_1.weight"] = (H, cfg.sincos_dim)
    t["time_guidance_embed.timestep_embedder.linear_2.weight"] = (H, H)
    t["double_stream_modulation_img.linear.weight"] = (6 * H, H)
    t["double_stream_modulation_txt.linear.weight"] = (6 * H, H)
    t["single_stream_modulation.linear.weight"] = (3 * H, H)
    for i in range(cfg.n_double):
        p = f"transformer_blocks.{i}."
        for n in ("norm_q", "norm_k", "norm_added_q", "norm_added_k"):
            t[p + f"attn.{n}.weight"] = (hd,)
        for n in ("to_q", "to_k", "to_v", "add_q_proj", "add_k_proj", "add_v_proj"):
            t[p + f"attn.{n}.weight"] = (H, H)
        t[p + "attn.to_out.0.weight"] = (H, H)
        t[p + "attn.to_add_out.weight"] = (H, H)
        t[p + "ff.linear_in.weight"] = (2 * M, H)
        t[p + "ff_context.linear_in.weight"] = (2 * M, H)
        t[p + "ff.linear_out.weight"] = (H, M)
        t[p + "ff_context.linear_out.weight"] = (H, M)
    for i in range(cfg.n_single):
        p = f"single_transformer_blocks.{i}."
        t[p + "attn.norm_q.weight"] = (hd,)
        t[p + "attn.norm_k.weight"] = (hd,)
        t[p + "attn.to_qkv_mlp_proj.weight"] = (3 * H + 2 * M, H)
        t[p + "attn.to_out.weight"] = (H, H + M)
    t["norm_out.linear.weight"] = (2 * H, H)
    t["proj_out.weight"] = (cfg.channels, H)
    return t


def is_qk_norm(name: str) -> bool:
    return ".attn.norm_" in name


_synth = None


def synth_lib():
    global _synth
    if _synth is None:
        path = os.path.join(_HERE, "libflux_synth.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is not built; run `python -c 'import __graft_entry__ as g; g.build()'`")
        lib = ctypes.CDLL(path)
        vp, i64, u64, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_uint64, ctypes.c_float
        lib.flux_synth_normal_f32.argtypes = [vp, i64, u64, u64, f32, f32]
        lib.flux_synth_normal_bf16.argtypes = [vp, i64, u64, u64, f32, f32]
        lib.flux_synth_fill_bf16.argtypes = [vp, i64, f32]
        lib.flux_synth_f32_to_bf16.argtypes = [vp, vp, i64]
        lib.flux_synth_bf16_to_f32.argtypes = [vp, vp, i64]
        for f in (lib.flux_synth_normal_f32, lib.flux_synth_normal_bf16, lib.flux_synth_fill_bf16,
                  lib.flux_synth_f32_to_bf16, lib.flux_synth_bf16_to_f32):
            f.restype = None
        _synth = lib
    return _synth


def normal_f32(shape, seed, stream, mean=0.0, std=1.0):
    out = np.empty(shape, dtype=np.float32)
    synth_lib().flux_synth_normal_f32(out.ctypes.data, out.size, seed, stream, mean, std)
    return out


def normal_bf16(shape, seed, stream, mean=0.0, std=1.0):
    out = np.empty(shape, dtype=np.uint16)
    synth_lib().flux_synth_normal_bf16(out.ctypes.data, out.size, seed, stream, mean, std)
    return out


def f32_to_bf16(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    synth_lib().flux_synth_f32_to_bf16(out.ctypes.data, x.ctypes.data, x.size)
    return out


def bf16_to_f32(x):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, dtype=np.float32)
    synth_lib().flux_synth_bf16_to_f32(out.ctypes.data, x.ctypes.data, x.size)
    return out


def make_weights(cfg: FluxConfig, seed=42, std=0.02, qk_norm="literal", only=None):
    """bf16 weights (uint16 arrays) keyed by tensor name.

    qk_norm="literal": the [head_dim] QK-norm weights are N(0, std) like every other tensor.
    qk_norm="sharp":   they are 1.0 (the usual RMSNorm initialisation), which gives attention
                       logits of order one so that RoPE/QK-norm/softmax errors become visible.
    """
    out = OrderedDict()
    for idx, (name, shape) in enumerate(tensor_shapes(cfg).items()):
        if only is not None and name not in only:
            continue
        if is_qk_norm(name) and qk_norm == "sharp":
            a = np.empty(shape, dtype=np.uint16)
            synth_lib().flux_synth_fill_bf16(a.ctypes.data, a.size, 1.0)
        else:
            a = normal_bf16(shape, seed, idx, 0.0, std)
        out[name] = a
    return out


def write_safetensors(path, tensors):
    """Minimal safetensors writer for bf16 tensors (format: flux_safetensors.h:4-8)."""
    import json
    header = {}
    off = 0
    for name, a in tensors.items():
        nb = a.size * 2
        header[name] = {"dtype": "BF16", "shape": list(a.shape), "data_offsets": [off, off + nb]}
        off += nb
    hj = json.dumps(header, separators=(",", ":")).encode()
    hj += b" " * ((8 - len(hj) % 8) % 8)
    with open(path, "wb") as f:
        f.write(len(hj).to_bytes(8, "little"))
        f.write(hj)
        for a in tensors.values():
            f.write(np.ascontiguousarray(a).tobytes())


def vae_tensor_shapes() -> "OrderedDict[str, tuple]":
    """Tensor names and shapes of the FLUX.2 VAE file as the reference reads it
    (flux_vae_load_safetensors, flux_vae.c:1232-1340): z 32 channels, base 128, multipliers 1,2,4,4,
    two residual blocks per encoder level and three per decoder level, GroupNorm(32)."""
    t = OrderedDict()
    mult = [1, 2, 4, 4]

    def conv(name, o, i, k):
        t[name + ".weight"] = (o, i, k, k)
        t[name + ".bias"] = (o,)

    def norm(name, c):
        t[name + ".weight"] = (c,)
        t[name + ".bias"] = (c,)

    def res(prefix, i, o):
        norm(prefix + ".norm1", i)
        conv(prefix + ".conv1", o, i, 3)
        norm(prefix + ".norm2", o)
        conv(prefix + ".conv2", o, o, 3)
        if i != o:
            conv(prefix + ".conv_shortcut", o, i, 1)

    def attn(prefix, c):
        norm(prefix + ".group_norm", c)
        for n in ("to_q", "to_k", "to_v", "to_out.0"):
            t[f"{prefix}.{n}.weight"] = (c, c)
            t[f"{prefix}.{n}.bias"] = (c,)

    conv("encoder.conv_in", 128, 3, 3)
    for lvl in range(4):
        ch = 128 * mult[lvl]
        prev = 128 if lvl == 0 else 128 * mult[lvl - 1]
        for r in range(2):
            res(f"encoder.down_blocks.{lvl}.resnets.{r}", prev if (r == 0 and lvl > 0) else ch, ch)
        if lvl < 3:
            conv(f"encoder.down_blocks.{lvl}.downsamplers.0.conv", ch, ch, 3)
    for side in ("encoder", "decoder"):
        res(f"{side}.mid_block.resnets.0", 512, 512)
        attn(f"{side}.mid_block.attentions.0", 512)
        res(f"{side}.mid_block.resnets.1", 512, 512)
    norm("encoder.conv_norm_out", 512)
    conv("encoder.conv_out", 64, 512, 3)
    conv("quant_conv", 64, 64, 1)
    conv("decoder.conv_in", 512, 32, 3)
    for up in range(4):
        lvl = 3 - up
        ch = 128 * mult[lvl]
        prev = 512 if lvl == 3 else 128 * mult[lvl + 1]
        for r in range(3):
            res(f"decoder.up_blocks.{up}.resnets.{r}", prev if r == 0 else ch, ch)
        if up < 3:
            conv(f"decoder.up_blocks.{up}.upsamplers.0.conv", ch, ch, 3)
    norm("decoder.conv_norm_out", 128)
    conv("decoder.conv_out", 3, 128, 3)
    t["bn.running_mean"] = (128,)
    t["bn.running_var"] = (128,)
    conv("post_quant_conv", 32, 32, 1)
    return t


def make_vae_weights(seed=77):
    """Synthetic bf16 VAE: convolution and linear weights ~N(0, 1/sqrt(fan_in)), norm scales near 1,
    small biases, positive running variances; enough for the decoder to give a textured image."""
    out = OrderedDict()
    for i, (name, shape) in enumerate(vae_tensor_shapes().items()):
        if name == "bn.running_var":
            out[name] = f32_to_bf16(1.0 + 0.2 * np.abs(normal_f32(shape, seed, 5000 + i)))
        elif name.endswith(".bias") or name == "bn.running_mean":
            out[name] = normal_bf16(shape, seed, 5000 + i, 0.0, 0.05)
        elif len(shape) == 1:
            out[name] = normal_bf16(shape, seed, 5000 + i, 1.0, 0.1)
        else:
            fan_in = int(np.prod(shape[1:]))
            out[name] = normal_bf16(shape, seed, 5000 + i, 0.0, 1.0 / np.sqrt(fan_in))
    return out


def vae_test_image(H, W, seed):
    """[3, H, W] in [-1, 1]: a smooth ramp plus noise, so that the VAE encoder sees structure and texture."""
    yy, xx = np.meshgrid(np.linspace(-1, 1, H, dtype=np.float32), np.linspace(-1, 1, W, dtype=np.float32), indexing="ij")
    base = np.stack([yy, xx, -0.5 * (yy + xx)]).astype(np.float32)
    return np.clip(0.6 * base + normal_f32((3, H, W), seed, 1, 0.0, 0.3), -1.0, 1.0).astype(np.float32)


def vae_decode_convs(h, w):
    """The decoder's convolutions for an h x w latent, in execution order (flux_vae_decode,
    flux_vae.c:690-837): (name, H, W, cin, cout, taps). All but the first (which the device folds into
    its input kernel) are one flux_hip_conv launch each, in this order."""
    mult = [1, 2, 4, 4]
    H, W = 2 * h, 2 * w
    out = [("post_quant_conv", H, W, 32, 32, 1), ("conv_in", H, W, 32, 512, 9)]

    def res(name, i, o):
        out.append((name + ".conv1", H, W, i, o, 9))
        if i != o:
            out.append((name + ".conv_shortcut", H, W, i, o, 1))
        out.append((name + ".conv2", H, W, o, o, 9))

    res("mid.0", 512, 512)
    out.append(("mid.attn.to_qkv", H, W, 512, 1536, 1))      # q, k and v projections, one launch on the device
    out.append(("mid.attn.to_out", H, W, 512, 512, 1))
    res("mid.1", 512, 512)
    prev = 512
    for up in range(4):
        ch = 128 * mult[3 - up]
        for r in range(3):
            res(f"up.{up}.{r}", prev if r == 0 else ch, ch)
        if up < 3:
            H, W = 2 * H, 2 * W
            out.append((f"up.{up}.upsample", H, W, ch, ch, 9))
        prev = ch
    out.append(("conv_out", H, W, 128, 3, 9))
    return out


def vae_decode_flops(h, w):
    """Algorithmic FLOPs of one decode (1 MAC = 2 FLOP): convolutions over the real image and channel
    counts, plus the mid-block attention's two products over (2h * 2w) positions at width 512."""
    conv = sum(2.0 * H * W * ci * co * t for _, H, W, ci, co, t in vae_decode_convs(h, w))
    n = 4.0 * h * w
    return conv + 4.0 * n * n * 512


def vae_encode_convs(H, W):
    """The encoder's convolutions for an H x W image, in execution order (flux_vae_encode,
    flux_vae.c:320-443): (name, output H, output W, cin, cout, taps); one flux_hip_conv launch each,
    in this order."""
    mult = [1, 2, 4, 4]
    out = [("conv_in", H, W, 3, 128, 9)]

    def res(name, i, o):
        out.append((name + ".conv1", H, W, i, o, 9))
        if i != o:
            out.append((name + ".conv_shortcut", H, W, i, o, 1))
        out.append((name + ".conv2", H, W, o, o, 9))

    prev = 128
    for lvl in range(4):
        ch = 128 * mult[lvl]
        for r in range(2):
            res(f"down.{lvl}.{r}", prev if r == 0 else ch, ch)
        if lvl < 3:
            H, W = H // 2, W // 2
            out.append((f"down.{lvl}.downsample", H, W, ch, ch, 9))
        prev = ch
    res("mid.0", 512, 512)
    out.append(("mid.attn.to_qkv", H, W, 512, 1536, 1))
    out.append(("mid.attn.to_out", H, W, 512, 512, 1))
    res("mid.1", 512, 512)
    out.append(("conv_out", H, W, 512, 64, 9))
    out.append(("quant_conv", H, W, 64, 64, 1))
    return out


def vae_encode_flops(H, W):
    """Algorithmic FLOPs of one encode: convolutions over the real image and channel counts, plus the
    mid-block attention's two products over (H/8 * W/8) positions at width 512."""
    conv = sum(2.0 * h * w * ci * co * t for _, h, w, ci, co, t in vae_encode_convs(H, W))
    n = (H // 8) * (W // 8)
    return conv + 4.0 * n * n * 512


@dataclass(frozen=True)
class QwenConfig:
    """Qwen3 text encoder (flux_qwen3.h:22-39): the hidden states after three layers, side by side,
    are the transformer's text input."""
    hidden: int = 2560
    intermediate: int = 9728
    heads: int = 32
    kv_heads: int = 8
    head_dim: int = 128
    layers: int = 36
    vocab: int = 151936
    out_layers: tuple = (8, 17, 26)
    rope_theta: float = 1000000.0
    eps: float = 1e-6


QWEN3_4B = QwenConfig()
# structurally identical, small enough for the CPU oracle to run in milliseconds
QWEN3_TINY = QwenConfig(hidden=256, intermediate=384, heads=4, kv_heads=2, layers=5, vocab=300, out_layers=(1, 2, 4))


def qwen3_tensor_shapes(cfg: QwenConfig) -> "OrderedDict[str, tuple]":
    """Tensor names and shapes as the reference loader reads them (flux_qwen3.c:1211-1253, 1361, 1376)."""
    t = OrderedDict()
    H, I, QD, KD = cfg.hidden, cfg.intermediate, cfg.heads * cfg.head_dim, cfg.kv_heads * cfg.head_dim
    t["model.embed_tokens.weight"] = (cfg.vocab, H)
    for i in range(cfg.layers):
        p = f"model.layers.{i}."
        t[p + "input_layernorm.weight"] = (H,)
        t[p + "post_attention_layernorm.weight"] = (H,)
        t[p + "self_attn.q_proj.weight"] = (QD, H)
        t[p + "self_attn.k_proj.weight"] = (KD, H)
        t[p + "self_attn.v_proj.weight"] = (KD, H)
        t[p + "self_attn.o_proj.weight"] = (H, QD)
        t[p + "self_attn.q_norm.weight"] = (cfg.head_dim,)
        t[p + "self_attn.k_norm.weight"] = (cfg.head_dim,)
        t[p + "mlp.gate_proj.weight"] = (I, H)
        t[p + "mlp.up_proj.weight"] = (I, H)
        t[p + "mlp.down_proj.weight"] = (H, I)
    t["model.norm.weight"] = (H,)
    return t


def make_qwen3_weights(cfg: QwenConfig, seed=61, only=None):
    """Synthetic bf16 encoder: projections ~N(0, 1/sqrt(fan_in)) (activations stay of order one through the
    layers), norm weights ~N(1, 0.1), embeddings ~N(0, 1)."""
    out = OrderedDict()
    for idx, (name, shape) in enumerate(qwen3_tensor_shapes(cfg).items()):
        if only is not None and name not in only:
            continue
        if len(shape) == 1:
            out[name] = normal_bf16(shape, seed, 9000 + idx, 1.0, 0.1)
        elif name == "model.embed_tokens.weight":
            out[name] = normal_bf16(shape, seed, 9000 + idx, 0.0, 1.0)
        else:
            out[name] = normal_bf16(shape, seed, 9000 + idx, 0.0, 1.0 / np.sqrt(shape[1]))
    return out


def qwen3_flops(cfg: QwenConfig, seq):
    """Algorithmic FLOPs of one encoder forward over seq tokens: the layers up to the last captured one;
    attention counted over the full seq x seq score matrix, as the reference computes it."""
    H, I, QD, KD = cfg.hidden, cfg.intermediate, cfg.heads * cfg.head_dim, cfg.kv_heads * cfg.head_dim
    n_layers = max(cfg.out_layers) + 1
    per_tok = 2.0 * (H * (QD + 2 * KD) + QD * H + 3 * H * I)
    return n_layers * (seq * per_tok + 4.0 * seq * seq * QD)


def flops_per_forward(cfg: FluxConfig, n_img, n_txt, n_img_out=None):
    """Algorithmic FLOPs of one forward (1 MAC = 2 FLOP)."""
    H, C, T = cfg.hidden, cfg.channels, cfg.text_dim
    n = n_img + n_txt
    n_out = n_img if n_img_out is None else n_img_out
    per_block = (2 * n * H * (3 * H + 2 * cfg.mlp) + 2 * n * (H + cfg.mlp) * H) + 4 * n * n * H
    return (cfg.n_double + cfg.n_single) * per_block + 2 * n_img * C * H + 2 * n_txt * T * H + 2 * n_out * H * C
