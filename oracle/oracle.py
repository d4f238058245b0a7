"""ctypes front-end of the CPU oracle (oracle/flux_oracle.c).

Test infrastructure only: the shipped backend never imports this module.
"""
import ctypes
import glob
import os
import sys

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(_HERE), "flux2.c_amd"))
from model_spec import FluxConfig  # noqa: E402

c_f = ctypes.c_float
c_i = ctypes.c_int
vp = ctypes.c_void_p


class _Cfg(ctypes.Structure):
    _fields_ = [(n, c_i) for n in ("hidden", "heads", "head_dim", "mlp", "n_double", "n_single",
                                   "text_dim", "channels", "axis_dim", "sincos_dim")] + [("rope_theta", c_f)]


class _Ref(ctypes.Structure):
    _fields_ = [("latent", vp), ("h", c_i), ("w", c_i), ("t_offset", c_i)]


class _QwenCfg(ctypes.Structure):
    _fields_ = [(n, c_i) for n in ("hidden", "intermediate", "heads", "kv_heads", "head_dim", "layers", "vocab")] + \
               [("out_layer", c_i * 3), ("rope_theta", c_f), ("eps", c_f)]


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    path = os.path.join(_HERE, "libflux_oracle.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is not built (make -C oracle)")
    L = ctypes.CDLL(path)
    L.fo_set_blas.argtypes = [ctypes.c_char_p, ctypes.c_char_p]
    L.fo_set_blas.restype = c_i
    L.fo_set_blas_threads.argtypes = [c_i]
    L.fo_model_new.argtypes = [ctypes.POINTER(_Cfg)]
    L.fo_model_new.restype = vp
    L.fo_model_free.argtypes = [vp]
    L.fo_model_set_bf16.argtypes = [vp, ctypes.c_char_p, vp, ctypes.c_int64]
    L.fo_model_set_bf16.restype = c_i
    L.fo_forward.argtypes = [vp, vp, c_i, c_i, vp, c_i, vp, c_i, c_f]
    L.fo_forward.restype = vp
    L.fo_free.argtypes = [vp]
    L.fo_sample_euler.argtypes = [vp, vp, c_i, c_i, vp, c_i, vp, c_i, vp, c_i, vp]
    L.fo_sample_euler.restype = vp
    L.fo_sample_euler_cfg.argtypes = [vp, vp, c_i, c_i, vp, c_i, vp, c_i, vp, c_i, c_f, vp, c_i, vp]
    L.fo_sample_euler_cfg.restype = vp
    L.fo_sample_heun.argtypes = [vp, vp, c_i, c_i, vp, c_i, vp, c_i, vp]
    L.fo_sample_heun.restype = vp
    L.fo_sample_euler_ancestral.argtypes = [vp, vp, c_i, c_i, vp, c_i, vp, c_i, c_f, vp]
    L.fo_sample_euler_ancestral.restype = vp
    L.fo_double_block.argtypes = [vp, c_i, vp, vp, vp, vp, vp, vp, vp, vp, c_i, c_i]
    L.fo_single_block.argtypes = [vp, c_i, vp, vp, vp, vp, vp, vp, c_i, c_i]
    L.fo_timestep_embedding.argtypes = [vp, c_f, c_i, c_f]
    L.fo_time_mlp.argtypes = [vp, vp, vp, vp, c_i, c_i]
    L.fo_rope_image.argtypes = [vp, vp, c_i, c_i, c_i, c_f, c_i]
    L.fo_rope_text.argtypes = [vp, vp, c_i, c_i, c_f]
    L.fo_apply_rope.argtypes = [vp, vp, vp, c_i, c_i, c_i]
    L.fo_adaln.argtypes = [vp, vp, vp, vp, c_i, c_i, c_f]
    L.fo_qk_norm.argtypes = [vp, vp, vp, vp, c_i, c_i, c_i, c_f]
    L.fo_linear.argtypes = [vp, vp, vp, c_i, c_i, c_i]
    L.fo_attention.argtypes = [vp, vp, vp, vp, c_i, c_i, c_i, c_i]
    L.fo_silu.argtypes = [vp, ctypes.c_int64]
    L.fo_softmax.argtypes = [vp, c_i, c_i]
    L.fo_gated_add.argtypes = [vp, vp, vp, c_i, c_i]
    L.fo_linear_schedule.argtypes = [vp, c_i]
    L.fo_power_schedule.argtypes = [vp, c_i, c_f]
    L.fo_official_schedule.argtypes = [vp, c_i, c_i]
    L.fo_sigmoid_schedule.argtypes = [vp, c_i, c_f]
    L.fo_resolution_schedule.argtypes = [vp, c_i, c_i, c_i]
    L.fo_init_noise.argtypes = [vp, c_i, c_i, c_i, ctypes.c_int64]
    L.fo_rng_seed.argtypes = [ctypes.c_uint64]
    L.fo_randn.argtypes = [vp, ctypes.c_int64]
    L.fo_num_threads.restype = c_i
    L.fo_has_blas.restype = c_i
    L.fo_conv2d.argtypes = [vp, vp, vp, vp, c_i, c_i, c_i, c_i, c_i, c_i]
    L.fo_group_norm.argtypes = [vp, vp, vp, vp, c_i, c_i, c_i, c_i, c_f]
    L.fo_upsample_nearest.argtypes = [vp, vp, c_i, c_i, c_i]
    L.fo_unpatchify.argtypes = [vp, vp, c_i, c_i, c_i, c_i]
    L.fo_patchify.argtypes = [vp, vp, c_i, c_i, c_i, c_i]
    L.fo_conv2d_down.argtypes = [vp, vp, vp, vp, c_i, c_i, c_i, c_i]
    L.fo_vae_encode.argtypes = [vp, vp, c_i, c_i, vp]
    L.fo_vae_encode.restype = c_i
    L.fo_vae_set_reference_aliasing.argtypes = [vp, c_i]
    L.fo_vae_new.argtypes = [c_i]
    L.fo_vae_new.restype = vp
    L.fo_vae_free.argtypes = [vp]
    L.fo_vae_set.argtypes = [vp, ctypes.c_char_p, vp, ctypes.c_int64]
    L.fo_vae_set.restype = c_i
    L.fo_vae_decode.argtypes = [vp, vp, c_i, c_i, vp, vp]
    L.fo_vae_decode.restype = c_i
    L.fo_qwen3_new.argtypes = [ctypes.POINTER(_QwenCfg)]
    L.fo_qwen3_new.restype = vp
    L.fo_qwen3_free.argtypes = [vp]
    L.fo_qwen3_set_bf16.argtypes = [vp, ctypes.c_char_p, vp, ctypes.c_int64]
    L.fo_qwen3_set_bf16.restype = c_i
    L.fo_qwen3_forward.argtypes = [vp, vp, vp, c_i]
    L.fo_qwen3_forward.restype = vp
    L.fo_qwen3_layer_forward.argtypes = [vp, c_i, vp, vp, c_i]
    L.fo_qwen3_rms_norm.argtypes = [vp, vp, vp, c_i, c_i, c_f]
    L.fo_qwen3_rope.argtypes = [vp, c_i, c_i, c_i, c_f]
    L.fo_qwen3_attention.argtypes = [vp, vp, vp, vp, vp, c_i, c_i, c_i, c_i]
    _lib = L
    return L


def enable_blas(threads=None):
    """Route the oracle's GEMMs through SciPy's bundled OpenBLAS when it is present.

    Returns the library path used, or None (then the built-in OpenMP loops run)."""
    L = lib()
    try:
        import scipy
        cands = glob.glob(os.path.join(os.path.dirname(scipy.__file__), "..", "scipy.libs", "libscipy_openblas*.so"))
    except Exception:
        cands = []
    for p in cands:
        if L.fo_set_blas(os.path.realpath(p).encode(), b"scipy_cblas_sgemm"):
            if threads:
                L.fo_set_blas_threads(int(threads))
            return p
    return None


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _make_refs(refs):
    if not refs:
        return None, 0, []
    keep = []
    arr = (_Ref * len(refs))()
    for i, (lat, h, w, toff) in enumerate(refs):
        lat = _f32(lat)
        keep.append(lat)
        arr[i] = _Ref(lat.ctypes.data, h, w, toff)
    return arr, len(refs), keep


class Oracle:
    """A loaded model. `weights` maps tensor name -> uint16 (bf16) array."""

    def __init__(self, cfg: FluxConfig, weights):
        self.cfg = cfg
        L = lib()
        c = _Cfg(cfg.hidden, cfg.heads, cfg.head_dim, cfg.mlp, cfg.n_double, cfg.n_single,
                 cfg.text_dim, cfg.channels, cfg.axis_dim, cfg.sincos_dim, cfg.rope_theta)
        self.h = L.fo_model_new(ctypes.byref(c))
        for name, a in weights.items():
            a = np.ascontiguousarray(a, dtype=np.uint16)
            rc = L.fo_model_set_bf16(self.h, name.encode(), a.ctypes.data, a.size)
            if rc != 0:
                raise ValueError(f"oracle rejected tensor {name}: rc={rc}")

    def close(self):
        if self.h:
            lib().fo_model_free(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _take(self, ptr, n):
        out = np.ctypeslib.as_array(ctypes.cast(ptr, ctypes.POINTER(c_f)), shape=(n,)).copy()
        lib().fo_free(ptr)
        return out

    def forward(self, latent, h, w, txt, t, refs=None):
        latent, txt = _f32(latent), _f32(txt)
        arr, n, keep = _make_refs(refs)
        p = lib().fo_forward(self.h, latent.ctypes.data, h, w, arr, n, txt.ctypes.data, txt.shape[0], t)
        return self._take(p, self.cfg.channels * h * w).reshape(self.cfg.channels, h, w)

    def sample_euler(self, z, h, w, txt, schedule, refs=None, trace=False):
        z, txt, schedule = _f32(z), _f32(txt), _f32(schedule)
        steps = len(schedule) - 1
        n = self.cfg.channels * h * w
        arr, nr, keep = _make_refs(refs)
        tr = np.zeros((steps, n), np.float32) if trace else None
        p = lib().fo_sample_euler(self.h, z.ctypes.data, h, w, arr, nr, txt.ctypes.data, txt.shape[0],
                                  schedule.ctypes.data, steps, tr.ctypes.data if trace else None)
        out = self._take(p, n).reshape(self.cfg.channels, h, w)
        return (out, tr) if trace else out

    def sample_euler_cfg(self, z, h, w, txt_cond, txt_uncond, guidance, schedule, refs=None, trace=False):
        z, tc, tu, schedule = _f32(z), _f32(txt_cond), _f32(txt_uncond), _f32(schedule)
        steps = len(schedule) - 1
        n = self.cfg.channels * h * w
        arr, nr, keep = _make_refs(refs)
        tr = np.zeros((2 * steps, n), np.float32) if trace else None
        p = lib().fo_sample_euler_cfg(self.h, z.ctypes.data, h, w, arr, nr, tc.ctypes.data, tc.shape[0],
                                      tu.ctypes.data, tu.shape[0], guidance, schedule.ctypes.data, steps,
                                      tr.ctypes.data if trace else None)
        out = self._take(p, n).reshape(self.cfg.channels, h, w)
        return (out, tr) if trace else out

    def sample_heun(self, z, h, w, txt, schedule, trace=False):
        """Heun sampler; the trace holds v1, v2 of every step in call order (2*steps - 1 rows)."""
        z, txt, schedule = _f32(z), _f32(txt), _f32(schedule)
        steps = len(schedule) - 1
        n = self.cfg.channels * h * w
        tr = np.zeros((max(2 * steps - 1, 0), n), np.float32) if trace else None
        p = lib().fo_sample_heun(self.h, z.ctypes.data, h, w, txt.ctypes.data, txt.shape[0],
                                 schedule.ctypes.data, steps, tr.ctypes.data if trace else None)
        out = self._take(p, n).reshape(self.cfg.channels, h, w)
        return (out, tr) if trace else out

    def sample_euler_ancestral(self, z, h, w, txt, schedule, eta, seed=None, trace=False):
        """Euler with noise injection; `seed` (if given) seeds the oracle's generator first."""
        z, txt, schedule = _f32(z), _f32(txt), _f32(schedule)
        steps = len(schedule) - 1
        n = self.cfg.channels * h * w
        if seed is not None:
            lib().fo_rng_seed(seed)
        tr = np.zeros((steps, n), np.float32) if trace else None
        p = lib().fo_sample_euler_ancestral(self.h, z.ctypes.data, h, w, txt.ctypes.data, txt.shape[0],
                                            schedule.ctypes.data, steps, eta, tr.ctypes.data if trace else None)
        out = self._take(p, n).reshape(self.cfg.channels, h, w)
        return (out, tr) if trace else out

    def double_block(self, idx, img_h, txt_h, img_mod, txt_mod, img_cos, img_sin, txt_cos, txt_sin):
        img_h, txt_h = _f32(img_h).copy(), _f32(txt_h).copy()
        a = [_f32(x) for x in (img_mod, txt_mod, img_cos, img_sin, txt_cos, txt_sin)]
        lib().fo_double_block(self.h, idx, img_h.ctypes.data, txt_h.ctypes.data, *[x.ctypes.data for x in a],
                              img_h.shape[0], txt_h.shape[0])
        return img_h, txt_h

    def single_block(self, idx, x, mod, img_cos, img_sin, txt_cos, txt_sin, txt_seq):
        x = _f32(x).copy()
        a = [_f32(v) for v in (mod, img_cos, img_sin, txt_cos, txt_sin)]
        lib().fo_single_block(self.h, idx, x.ctypes.data, *[v.ctypes.data for v in a], x.shape[0], txt_seq)
        return x


# ---- stateless operators -------------------------------------------------

def timestep_embedding(t, dim=256, max_period=10000.0):
    out = np.empty(dim, np.float32)
    lib().fo_timestep_embedding(out.ctypes.data, t, dim, max_period)
    return out


def time_mlp(e, fc1, fc2):
    e, fc1, fc2 = _f32(e), _f32(fc1), _f32(fc2)
    out = np.empty(fc2.shape[0], np.float32)
    lib().fo_time_mlp(out.ctypes.data, e.ctypes.data, fc1.ctypes.data, fc2.ctypes.data, e.size, fc2.shape[0])
    return out


def rope_image(ph, pw, axis_dim=32, theta=2000.0, t_offset=0):
    c = np.empty((ph * pw, 4 * axis_dim), np.float32)
    s = np.empty_like(c)
    lib().fo_rope_image(c.ctypes.data, s.ctypes.data, ph, pw, axis_dim, theta, t_offset)
    return c, s


def rope_text(seq, axis_dim=32, theta=2000.0):
    c = np.empty((seq, 4 * axis_dim), np.float32)
    s = np.empty_like(c)
    lib().fo_rope_text(c.ctypes.data, s.ctypes.data, seq, axis_dim, theta)
    return c, s


def apply_rope(x, cos, sin, heads, head_dim):
    x = _f32(x).copy()
    cos, sin = _f32(cos), _f32(sin)
    lib().fo_apply_rope(x.ctypes.data, cos.ctypes.data, sin.ctypes.data, x.shape[0], heads, head_dim)
    return x


def adaln(x, shift, scale, eps=1e-6):
    x, shift, scale = _f32(x), _f32(shift), _f32(scale)
    out = np.empty_like(x)
    lib().fo_adaln(out.ctypes.data, x.ctypes.data, shift.ctypes.data, scale.ctypes.data, x.shape[0], x.shape[1], eps)
    return out


def qk_norm(q, k, qw, kw, heads, head_dim, eps=1e-6):
    q, k = _f32(q).copy(), _f32(k).copy()
    qw, kw = _f32(qw), _f32(kw)
    lib().fo_qk_norm(q.ctypes.data, k.ctypes.data, qw.ctypes.data, kw.ctypes.data, q.shape[0], heads, head_dim, eps)
    return q, k


def linear(x, W):
    x, W = _f32(x), _f32(W)
    y = np.empty((x.shape[0], W.shape[0]), np.float32)
    lib().fo_linear(y.ctypes.data, x.ctypes.data, W.ctypes.data, x.shape[0], x.shape[1], W.shape[0])
    return y


def attention(q, k, v, heads, head_dim):
    q, k, v = _f32(q), _f32(k), _f32(v)
    out = np.empty_like(q)
    lib().fo_attention(out.ctypes.data, q.ctypes.data, k.ctypes.data, v.ctypes.data, q.shape[0], k.shape[0], heads, head_dim)
    return out


def silu(x):
    x = _f32(x).copy()
    lib().fo_silu(x.ctypes.data, x.size)
    return x


def softmax(x):
    x = _f32(x).copy()
    lib().fo_softmax(x.ctypes.data, x.shape[0], x.shape[1])
    return x


def gated_add(out, gate, proj):
    out, gate, proj = _f32(out).copy(), _f32(gate), _f32(proj)
    lib().fo_gated_add(out.ctypes.data, gate.ctypes.data, proj.ctypes.data, out.shape[0], out.shape[1])
    return out


def linear_schedule(n):
    s = np.empty(n + 1, np.float32)
    lib().fo_linear_schedule(s.ctypes.data, n)
    return s


def power_schedule(n, alpha):
    s = np.empty(n + 1, np.float32)
    lib().fo_power_schedule(s.ctypes.data, n, alpha)
    return s


def official_schedule(n, image_seq_len):
    s = np.empty(n + 1, np.float32)
    lib().fo_official_schedule(s.ctypes.data, n, image_seq_len)
    return s


def sigmoid_schedule(n, shift):
    s = np.empty(n + 1, np.float32)
    lib().fo_sigmoid_schedule(s.ctypes.data, n, shift)
    return s


def resolution_schedule(n, height, width):
    s = np.empty(n + 1, np.float32)
    lib().fo_resolution_schedule(s.ctypes.data, n, height, width)
    return s


def init_noise(channels, h, w, seed):
    out = np.empty((channels, h, w), np.float32)
    lib().fo_init_noise(out.ctypes.data, channels, h, w, seed)
    return out


def randn(n, seed):
    out = np.empty(n, np.float32)
    lib().fo_rng_seed(seed)
    lib().fo_randn(out.ctypes.data, n)
    return out


# ---- VAE decoder (oracle/vae_oracle.c) ----

def conv2d(x, w, bias, pad):
    """x [cin, H, W], w [cout, cin, k, k] -> [cout, H, W] (stride 1, zero padding)."""
    x, w = _f32(x), _f32(w)
    b = None if bias is None else _f32(bias)
    out = np.empty((w.shape[0], x.shape[1], x.shape[2]), np.float32)
    lib().fo_conv2d(out.ctypes.data, x.ctypes.data, w.ctypes.data, None if b is None else b.ctypes.data,
                    x.shape[0], w.shape[0], x.shape[1], x.shape[2], w.shape[2], pad)
    return out


def group_norm(x, gamma, beta, groups=32, eps=1e-4):
    x, gamma, beta = _f32(x), _f32(gamma), _f32(beta)
    out = np.empty_like(x)
    lib().fo_group_norm(out.ctypes.data, x.ctypes.data, gamma.ctypes.data, beta.ctypes.data,
                        x.shape[0], x.shape[1], x.shape[2], groups, eps)
    return out


def upsample_nearest(x):
    x = _f32(x)
    out = np.empty((x.shape[0], 2 * x.shape[1], 2 * x.shape[2]), np.float32)
    lib().fo_upsample_nearest(out.ctypes.data, x.ctypes.data, x.shape[0], x.shape[1], x.shape[2])
    return out


def unpatchify(x, p=2):
    x = _f32(x)
    c = x.shape[0] // (p * p)
    out = np.empty((c, p * x.shape[1], p * x.shape[2]), np.float32)
    lib().fo_unpatchify(out.ctypes.data, x.ctypes.data, c, x.shape[1], x.shape[2], p)
    return out


def patchify(x, p=2):
    """[C, H, W] -> [C*p*p, H/p, W/p]."""
    x = _f32(x)
    out = np.empty((x.shape[0] * p * p, x.shape[1] // p, x.shape[2] // p), np.float32)
    lib().fo_patchify(out.ctypes.data, x.ctypes.data, x.shape[0], x.shape[1], x.shape[2], p)
    return out


def conv2d_down(x, w, bias=None):
    """The encoder's downsampling convolution: x [cin, H, W] padded by one row below and one column on the
    right, 3x3 kernel w [cout, cin, 3, 3], stride 2."""
    x, w = _f32(x), _f32(w)
    b = None if bias is None else _f32(bias)
    H, W = x.shape[1], x.shape[2]
    out = np.empty((w.shape[0], (H - 2) // 2 + 1, (W - 2) // 2 + 1), np.float32)
    lib().fo_conv2d_down(out.ctypes.data, x.ctypes.data, w.ctypes.data, None if b is None else b.ctypes.data,
                         x.shape[0], w.shape[0], H, W)
    return out


class VaeOracle:
    """The VAE. `weights` maps tensor name -> uint16 (bf16) or float32 array."""

    def __init__(self, weights, base_channels=128):
        from model_spec import bf16_to_f32
        self._L = lib()
        self._v = self._L.fo_vae_new(base_channels)
        for name, a in weights.items():
            a = _f32(bf16_to_f32(a) if a.dtype == np.uint16 else a)
            rc = self._L.fo_vae_set(self._v, name.encode(), a.ctypes.data, a.size)
            if rc != 0:
                raise ValueError(f"vae oracle rejected tensor {name}")

    def close(self):
        if self._v:
            self._L.fo_vae_free(self._v)
            self._v = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def decode(self, latent, h, w):
        """latent [128, h, w] -> (float image [3, 16h, 16w] in about [-1, 1], uint8 image [16h, 16w, 3])."""
        latent = _f32(latent)
        f = np.empty((3, 16 * h, 16 * w), np.float32)
        u = np.empty((16 * h, 16 * w, 3), np.uint8)
        if self._L.fo_vae_decode(self._v, latent.ctypes.data, h, w, f.ctypes.data, u.ctypes.data) != 0:
            raise RuntimeError("vae oracle: decode failed (missing tensor)")
        return f, u

    def encode(self, img, reference_aliasing=False):
        """img [3, H, W] in [-1, 1], H and W multiples of 16 -> normalised latent [128, H/16, W/16].
        reference_aliasing: reproduce the buffer overlap of the reference's generic build in the two
        widening residual blocks (see resblock() in vae_oracle.c); only for checks against that build."""
        img = _f32(img)
        self._L.fo_vae_set_reference_aliasing(self._v, int(reference_aliasing))
        H, W = img.shape[1], img.shape[2]
        lat = np.empty((128, H // 16, W // 16), np.float32)
        if self._L.fo_vae_encode(self._v, img.ctypes.data, H, W, lat.ctypes.data) != 0:
            raise RuntimeError("vae oracle: encode failed (missing tensor or size not a multiple of 16)")
        return lat


# ---- Qwen3 text encoder (oracle/qwen3_oracle.c) ----

def qwen3_rms_norm(x, w, eps=1e-6):
    x, w = _f32(x), _f32(w)
    out = np.empty_like(x)
    lib().fo_qwen3_rms_norm(out.ctypes.data, x.ctypes.data, w.ctypes.data, x.shape[0], x.shape[1], eps)
    return out


def qwen3_rope(x, heads, head_dim, theta=1000000.0):
    """x [seq, heads*head_dim] -> rotated copy."""
    x = _f32(x).copy()
    lib().fo_qwen3_rope(x.ctypes.data, x.shape[0], heads, head_dim, theta)
    return x


def qwen3_attention(q, k, v, mask, heads, kv_heads, head_dim=128):
    """q [seq, heads*hd], k, v [seq, kv_heads*hd], mask int [seq] or None -> [seq, heads*hd]."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    m = None if mask is None else np.ascontiguousarray(mask, dtype=np.int32)
    out = np.empty_like(q)
    lib().fo_qwen3_attention(out.ctypes.data, q.ctypes.data, k.ctypes.data, v.ctypes.data, None if m is None else m.ctypes.data,
                             q.shape[0], heads, kv_heads, head_dim)
    return out


class Qwen3Oracle:
    """`weights` maps tensor name -> uint16 (bf16) array; cfg is a model_spec.QwenConfig."""

    def __init__(self, cfg, weights):
        self.cfg = cfg
        self._L = lib()
        c = _QwenCfg(cfg.hidden, cfg.intermediate, cfg.heads, cfg.kv_heads, cfg.head_dim, cfg.layers, cfg.vocab,
                     (c_i * 3)(*cfg.out_layers), cfg.rope_theta, cfg.eps)
        self._m = self._L.fo_qwen3_new(ctypes.byref(c))
        for name, a in weights.items():
            a = np.ascontiguousarray(a, dtype=np.uint16)
            rc = self._L.fo_qwen3_set_bf16(self._m, name.encode(), a.ctypes.data, a.size)
            if rc < 0:
                raise ValueError(f"qwen3 oracle rejected tensor {name}: {rc}")

    def close(self):
        if self._m:
            self._L.fo_qwen3_free(self._m)
            self._m = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def forward(self, ids, mask=None):
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        m = None if mask is None else np.ascontiguousarray(mask, dtype=np.int32)
        p = self._L.fo_qwen3_forward(self._m, ids.ctypes.data, None if m is None else m.ctypes.data, ids.size)
        n = ids.size * 3 * self.cfg.hidden
        out = np.ctypeslib.as_array(ctypes.cast(p, ctypes.POINTER(c_f)), shape=(n,)).copy().reshape(ids.size, 3 * self.cfg.hidden)
        self._L.fo_free(p)
        return out

    def layer(self, idx, h, mask=None):
        h = _f32(h).copy()
        m = None if mask is None else np.ascontiguousarray(mask, dtype=np.int32)
        self._L.fo_qwen3_layer_forward(self._m, idx, h.ctypes.data, None if m is None else m.ctypes.data, h.shape[0])
        return h
