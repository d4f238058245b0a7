"""ctypes binding of libflux_hip.so (include/flux_hip.h) for tests, the smoke entry and the benchmark.

This module only marshals numpy arrays to the C ABI. It contains no arithmetic of its own and
has no CPU fallback: if the library or a GPU is missing, calls raise.
"""
import ctypes
import os

import numpy as np

from model_spec import FluxConfig

_HERE = os.path.dirname(os.path.abspath(__file__))
c_f, c_i, vp, c_sz = ctypes.c_float, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t

EPI_BF16, EPI_F32, EPI_F32_T, EPI_RESID, EPI_SWIGLU = range(5)
EPI_CONV_BF16, EPI_CONV_F32 = 6, 7


class _Cfg(ctypes.Structure):
    _fields_ = [(n, c_i) for n in ("hidden", "heads", "head_dim", "mlp", "n_double", "n_single",
                                   "text_dim", "channels", "axis_dim", "sincos_dim")] + [("rope_theta", c_f)]


class _QwenCfg(ctypes.Structure):
    _fields_ = [(n, c_i) for n in ("hidden", "intermediate", "heads", "kv_heads", "head_dim", "layers", "vocab")] + \
               [("out_layer", c_i * 3), ("rope_theta", c_f), ("eps", c_f)]


class _Part(ctypes.Structure):
    _fields_ = [("A", vp), ("W", vp), ("C", vp), ("gate", vp), ("M", c_i)]


class _Ref(ctypes.Structure):
    _fields_ = [("latent", vp), ("h", c_i), ("w", c_i), ("t_offset", c_i)]


class FluxHipError(RuntimeError):
    pass


_lib = None


def lib_path():
    """libflux_hip.so next to this file, or the file FLUX_HIP_LIBRARY names (another build of the same ABI)."""
    return os.environ.get("FLUX_HIP_LIBRARY") or os.path.join(_HERE, "libflux_hip.so")


def lib():
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise FluxHipError(f"{path} is not built (make -C flux2.c_amd hip)")
    L = ctypes.CDLL(path)
    L.flux_hip_init.restype = c_i
    L.flux_hip_available.restype = c_i
    L.flux_hip_sync.restype = c_i
    L.flux_hip_last_error.restype = ctypes.c_char_p
    L.flux_hip_stream.restype = vp
    L.flux_hip_malloc.restype = vp
    L.flux_hip_malloc.argtypes = [c_sz]
    L.flux_hip_free.argtypes = [vp]
    L.flux_hip_upload.argtypes = [vp, vp, c_sz]
    L.flux_hip_download.argtypes = [vp, vp, c_sz]
    L.flux_hip_memset.argtypes = [vp, c_i, c_sz]
    L.flux_hip_timer_stop.restype = c_f
    L.flux_hip_linear.argtypes = [c_i, c_i, ctypes.POINTER(_Part), c_i, c_i, c_i, c_i, c_i, c_i, c_i]
    L.flux_hip_linear_force_tile.argtypes = [c_i]
    L.flux_hip_set_batched_cfg.argtypes = [c_i]
    L.flux_hip_linear_enable_splitk.argtypes = [c_i]
    L.flux_hip_linear_persistent.argtypes = [c_i]
    L.flux_hip_attention_force_variant.argtypes = [c_i]
    L.flux_hip_linear_probe.argtypes = [c_i]
    L.flux_hip_linear_probe_read.argtypes = [ctypes.POINTER(c_i), ctypes.POINTER(c_f)]
    L.flux_hip_linear_probe_read_tile.argtypes = [c_i, ctypes.POINTER(c_i), ctypes.POINTER(c_f)]
    L.flux_hip_linear_probe_read_launches.argtypes = [c_i, vp, vp]
    L.flux_hip_adaln_norm.argtypes = [vp, c_i, vp, c_i, c_i, c_i, vp, vp, vp, vp, c_f]
    L.flux_hip_qk_prepare.argtypes = [vp, vp, c_i, c_i, c_i, c_i, c_i, c_i, vp, vp, vp, vp, vp, vp, c_f]
    L.flux_hip_attention.argtypes = [vp, c_i, vp, c_i, vp, vp, c_i, c_i, c_i, c_i]
    L.flux_hip_attention_batch.argtypes = [c_i, vp, c_i, vp, c_i, vp, vp, c_i, vp, vp, c_i]
    L.flux_hip_gemv.argtypes = [vp, vp, vp, c_i, c_i, c_i, c_i]
    L.flux_hip_latent_to_tokens.argtypes = [vp, vp, c_i, c_i]
    L.flux_hip_f32_to_bf16.argtypes = [vp, vp, c_sz]
    L.flux_hip_euler_update.argtypes = [vp, vp, c_f, c_sz]
    L.flux_hip_cfg_euler_update.argtypes = [vp, vp, vp, c_f, c_f, c_sz]
    L.flux_hip_transformer_new.restype = vp
    L.flux_hip_transformer_new.argtypes = [ctypes.POINTER(_Cfg)]
    L.flux_hip_transformer_set_tensor.argtypes = [vp, ctypes.c_char_p, vp, ctypes.c_int64]
    L.flux_hip_transformer_load_file.restype = vp
    L.flux_hip_transformer_load_file.argtypes = [ctypes.c_char_p, ctypes.POINTER(_Cfg)]
    L.flux_transformer_free.argtypes = [vp]
    L.flux_transformer_forward.restype = vp
    L.flux_transformer_forward.argtypes = [vp, vp, c_i, c_i, vp, c_i, c_f]
    L.flux_transformer_forward_with_refs.restype = vp
    L.flux_transformer_forward_with_refs.argtypes = [vp, vp, c_i, c_i, vp, c_i, c_i, c_i, vp, c_i, c_f]
    L.flux_transformer_forward_with_multi_refs.restype = vp
    L.flux_transformer_forward_with_multi_refs.argtypes = [vp, vp, c_i, c_i, vp, c_i, vp, c_i, c_f]
    L.flux_hip_sample_traced.restype = vp
    L.flux_hip_sample_traced.argtypes = [vp, vp, c_i, c_i, c_i, vp, c_i, vp, c_i, vp, c_i, c_f, vp, c_i, vp]
    L.flux_sample_euler.restype = vp
    L.flux_sample_euler.argtypes = [vp, vp, vp, c_i, c_i, c_i, c_i, vp, c_i, vp, c_i, vp]
    L.flux_sample_euler_with_refs.restype = vp
    L.flux_sample_euler_with_refs.argtypes = [vp, vp, vp, c_i, c_i, c_i, c_i, vp, c_i, c_i, c_i, vp, c_i, vp, c_i, vp]
    L.flux_sample_euler_cfg.restype = vp
    L.flux_sample_euler_cfg.argtypes = [vp, vp, vp, c_i, c_i, c_i, c_i, vp, c_i, vp, c_i, c_f, vp, c_i, vp]
    L.flux_sample_euler_cfg_with_refs.restype = vp
    L.flux_sample_euler_cfg_with_refs.argtypes = [vp, vp, vp, c_i, c_i, c_i, c_i, vp, c_i, c_i, c_i,
                                                  vp, c_i, vp, c_i, c_f, vp, c_i, vp]
    L.flux_hip_session_begin.restype = vp
    L.flux_hip_session_begin.argtypes = [vp, vp, c_i, c_i, c_i, vp, c_i, vp, c_i, vp, c_i, c_f, vp, c_i]
    L.flux_hip_session_step.argtypes = [vp, c_i, vp]
    L.flux_hip_session_read_latent.argtypes = [vp, vp]
    L.flux_hip_session_free.argtypes = [vp]
    L.flux_init_noise.restype = vp
    L.flux_init_noise.argtypes = [c_i, c_i, c_i, c_i, ctypes.c_int64]
    for n in ("flux_linear_schedule", "flux_power_schedule", "flux_official_schedule", "flux_sigmoid_schedule",
              "flux_resolution_schedule", "flux_hip_sample_heun_traced", "flux_hip_sample_ancestral_traced",
              "flux_sample_heun", "flux_sample_euler_ancestral", "flux_generate_latent"):
        getattr(L, n).restype = vp
    L.flux_sigmoid_schedule.argtypes = [c_i, c_f]
    L.flux_resolution_schedule.argtypes = [c_i, c_i, c_i]
    L.flux_hip_sample_heun_traced.argtypes = [vp, vp, c_i, c_i, c_i, vp, c_i, vp, c_i, vp, vp]
    L.flux_hip_sample_ancestral_traced.argtypes = [vp, vp, c_i, c_i, c_i, vp, c_i, vp, c_i, c_f, vp, vp]
    L.flux_sample_heun.argtypes = [vp, vp, c_i, c_i, c_i, c_i, vp, c_i, vp, c_i, vp]
    L.flux_sample_euler_ancestral.argtypes = [vp, vp, c_i, c_i, c_i, c_i, vp, c_i, vp, c_i, c_f, vp]
    L.flux_generate_latent.argtypes = [vp, vp, c_i, c_i, c_i, c_i, ctypes.c_int64, vp]
    L.flux_rng_seed.argtypes = [ctypes.c_uint64]
    L.flux_rng_seed.restype = None
    L.flux_randn.argtypes = [vp, c_i]
    L.flux_randn.restype = None
    L.flux_linear_schedule.argtypes = [c_i]
    L.flux_power_schedule.argtypes = [c_i, c_f]
    L.flux_official_schedule.argtypes = [c_i, c_i]
    L.flux_hip_linear_resid_adaln.argtypes = [c_i, vp, c_i, c_i, c_i, c_i, c_i, vp, c_f, ctypes.POINTER(c_i)]
    L.flux_hip_conv.argtypes = [c_i, vp, vp, vp, vp, vp, c_i, c_i, c_i, c_i, c_i]
    L.flux_hip_group_norm.argtypes = [vp, vp, vp, c_i, vp, vp, vp, c_i, c_i, c_i, c_f, c_i]
    L.flux_hip_conv_stats.argtypes = [c_i, vp, vp, vp, vp, vp, c_i, c_i, c_i, c_i, c_i, vp, ctypes.POINTER(c_i)]
    L.flux_hip_group_norm_stats.argtypes = [vp, vp, vp, c_i, vp, vp, vp, c_i, c_i, c_i, c_f, c_i, vp, c_i]
    L.flux_hip_group_norm_scratch_floats.restype = c_sz
    L.flux_hip_group_norm_scratch_floats.argtypes = [c_i, c_i]
    L.flux_hip_upsample2x.argtypes = [vp, vp, c_i, c_i, c_i]
    L.flux_hip_softmax_rows.argtypes = [vp, vp, vp, c_i, c_i, c_f]
    L.flux_hip_transpose_bf16.argtypes = [vp, c_i, vp, c_i, c_i, c_i]
    L.flux_hip_vae_new.restype = vp
    L.flux_hip_vae_load_file.restype = vp
    L.flux_hip_vae_load_file.argtypes = [ctypes.c_char_p]
    L.flux_hip_vae_set_tensor.argtypes = [vp, ctypes.c_char_p, c_i, vp, ctypes.c_int64]
    L.flux_hip_vae_free.argtypes = [vp]
    L.flux_hip_vae_decode.argtypes = [vp, vp, c_i, c_i, vp, vp]
    L.flux_hip_vae_set_attention_chunk.argtypes = [c_i]
    L.flux_hip_vae_encode.argtypes = [vp, vp, c_i, c_i, vp]
    L.flux_hip_vae_image_in.argtypes = [vp, vp, c_i, c_i]
    L.flux_hip_downsample_gather.argtypes = [vp, vp, c_i, c_i, c_i]
    L.flux_hip_vae_latent_out.argtypes = [vp, vp, c_i, vp, vp, c_i, c_i, c_f]
    L.flux_hip_rms_norm.argtypes = [vp, vp, vp, c_i, c_i, c_f]
    L.flux_hip_causal_attention.argtypes = [vp, vp, vp, c_i, vp, c_i, c_i, c_i]
    L.flux_hip_qwen3_new.restype = vp
    L.flux_hip_qwen3_new.argtypes = [ctypes.POINTER(_QwenCfg)]
    L.flux_hip_qwen3_load_dir.restype = vp
    L.flux_hip_qwen3_load_dir.argtypes = [ctypes.c_char_p]
    L.flux_hip_qwen3_set_tensor.argtypes = [vp, ctypes.c_char_p, c_i, vp, ctypes.c_int64]
    L.flux_hip_qwen3_free.argtypes = [vp]
    L.flux_hip_qwen3_forward.restype = vp
    L.flux_hip_qwen3_forward.argtypes = [vp, vp, vp, c_i]
    _lib = L
    return L


def libc_free(ptr):
    ctypes.CDLL(None).free(ctypes.c_void_p(ptr))


def check(rc, what="flux_hip call"):
    if not rc:
        raise FluxHipError(f"{what} failed: {lib().flux_hip_last_error().decode()}")
    return rc


def init():
    check(lib().flux_hip_init(), "flux_hip_init")


def sync():
    check(lib().flux_hip_sync(), "flux_hip_sync")


class DevBuf:
    """A device allocation with numpy upload/download."""

    def __init__(self, nbytes):
        init()
        self.nbytes = int(nbytes)
        self.ptr = lib().flux_hip_malloc(self.nbytes)
        if not self.ptr:
            raise FluxHipError(f"flux_hip_malloc({nbytes}): {lib().flux_hip_last_error().decode()}")

    @classmethod
    def from_array(cls, a):
        a = np.ascontiguousarray(a)
        b = cls(max(a.nbytes, 1))
        if a.nbytes:
            check(lib().flux_hip_upload(b.ptr, a.ctypes.data, a.nbytes), "upload")
        return b

    def to_array(self, dtype, shape):
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        if out.nbytes:
            check(lib().flux_hip_download(out.ctypes.data, self.ptr, out.nbytes), "download")
        return out

    def at(self, byte_offset):
        return self.ptr + int(byte_offset)

    def free(self):
        if self.ptr:
            lib().flux_hip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def linear(epilogue, parts, N, K, lda, ldw, ldc, w_row0=0, w_row1=0):
    """parts: list of (A_ptr, W_ptr, C_ptr, gate_ptr_or_None, M)."""
    arr = (_Part * len(parts))()
    for i, (A, W, C, g, M) in enumerate(parts):
        arr[i] = _Part(A, W, C, g, M)
    check(lib().flux_hip_linear(epilogue, len(parts), arr, N, K, lda, ldw, ldc, w_row0, w_row1), "flux_hip_linear")


class _AdalnPart(ctypes.Structure):
    _fields_ = [("out_bf16", vp), ("shift", vp), ("scale", vp)]


def linear_resid_adaln(parts, N, K, lda, ldw, ldc, norms, eps=1e-6):
    """parts as for linear() with the residual epilogue; norms: list of (out_bf16_ptr, shift_ptr, scale_ptr) per
    part, or None. Returns True when the AdaLN outputs were written (the projection ran as K slices)."""
    arr = (_Part * len(parts))()
    for i, (A, W, C, g, M) in enumerate(parts):
        arr[i] = _Part(A, W, C, g, M)
    na = None
    if norms is not None:
        na = (_AdalnPart * len(parts))()
        for i, (o, sh, sc) in enumerate(norms):
            na[i] = _AdalnPart(o, sh, sc)
    fused = c_i(0)
    check(lib().flux_hip_linear_resid_adaln(len(parts), arr, N, K, lda, ldw, ldc, na, eps, ctypes.byref(fused)), "flux_hip_linear_resid_adaln")
    return bool(fused.value)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _refs_array(refs):
    if not refs:
        return None, 0, []
    keep = []
    arr = (_Ref * len(refs))()
    for i, (lat, h, w, t) in enumerate(refs):
        lat = _f32(lat)
        keep.append(lat)
        arr[i] = _Ref(lat.ctypes.data, h, w, t)
    return arr, len(refs), keep


def _take_host(ptr, shape):
    n = int(np.prod(shape))
    out = np.ctypeslib.as_array(ctypes.cast(ptr, ctypes.POINTER(c_f)), shape=(n,)).copy().reshape(shape)
    libc_free(ptr)
    return out


class Transformer:
    """The denoising transformer on the GPU, built from named bf16 tensors or a safetensors file."""

    def __init__(self, cfg: FluxConfig, weights=None, path=None):
        init()
        self.cfg = cfg
        L = lib()
        c = _Cfg(cfg.hidden, cfg.heads, cfg.head_dim, cfg.mlp, cfg.n_double, cfg.n_single, cfg.text_dim,
                 cfg.channels, cfg.axis_dim, cfg.sincos_dim, cfg.rope_theta)
        if path is not None:
            self.h = L.flux_hip_transformer_load_file(os.fsencode(path), ctypes.byref(c))
            if not self.h:
                raise FluxHipError(f"load_file: {L.flux_hip_last_error().decode()}")
            return
        self.h = L.flux_hip_transformer_new(ctypes.byref(c))
        if not self.h:
            raise FluxHipError(f"transformer_new: {L.flux_hip_last_error().decode()}")
        if weights:
            for name, a in weights.items():
                self.set_tensor(name, a)

    def set_tensor(self, name, a):
        a = np.ascontiguousarray(a, dtype=np.uint16)
        check(lib().flux_hip_transformer_set_tensor(self.h, name.encode(), a.ctypes.data, a.size), f"set_tensor({name})")

    def close(self):
        if getattr(self, "h", None):
            lib().flux_transformer_free(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def forward(self, latent, h, w, txt, t, refs=None):
        latent, txt = _f32(latent), _f32(txt)
        arr, n, keep = _refs_array(refs)
        L = lib()
        if n == 0:
            p = L.flux_transformer_forward(self.h, latent.ctypes.data, h, w, txt.ctypes.data, txt.shape[0], t)
        elif n == 1:
            r = arr[0]
            p = L.flux_transformer_forward_with_refs(self.h, latent.ctypes.data, h, w, r.latent, r.h, r.w, r.t_offset,
                                                     txt.ctypes.data, txt.shape[0], t)
        else:
            p = L.flux_transformer_forward_with_multi_refs(self.h, latent.ctypes.data, h, w, arr, n,
                                                           txt.ctypes.data, txt.shape[0], t)
        if not p:
            raise FluxHipError(f"forward: {L.flux_hip_last_error().decode()}")
        return _take_host(p, (self.cfg.channels, h, w))

    def sample(self, z, h, w, txt, schedule, refs=None, txt_uncond=None, guidance=0.0, trace=False):
        """Euler (or CFG when txt_uncond is given) sampling loop on the device."""
        z, txt, schedule = _f32(z), _f32(txt), _f32(schedule)
        steps = len(schedule) - 1
        n = self.cfg.channels * h * w
        arr, nr, keep = _refs_array(refs)
        tu = _f32(txt_uncond) if txt_uncond is not None else None
        fw = steps * (2 if tu is not None else 1)
        tr = np.zeros((fw, n), np.float32) if trace else None
        L = lib()
        p = L.flux_hip_sample_traced(self.h, z.ctypes.data, self.cfg.channels, h, w, arr, nr,
                                     txt.ctypes.data, txt.shape[0],
                                     tu.ctypes.data if tu is not None else None, tu.shape[0] if tu is not None else 0,
                                     guidance, schedule.ctypes.data, steps, tr.ctypes.data if trace else None)
        if not p:
            raise FluxHipError(f"sample: {L.flux_hip_last_error().decode()}")
        out = _take_host(p, (self.cfg.channels, h, w))
        return (out, tr) if trace else out


    def sample_heun(self, z, h, w, txt, schedule, trace=False):
        """Heun sampling loop; the trace holds v1, v2 of every step in call order (2*steps - 1 rows)."""
        z, txt, schedule = _f32(z), _f32(txt), _f32(schedule)
        steps = len(schedule) - 1
        n = self.cfg.channels * h * w
        tr = np.zeros((max(2 * steps - 1, 0), n), np.float32) if trace else None
        L = lib()
        p = L.flux_hip_sample_heun_traced(self.h, z.ctypes.data, self.cfg.channels, h, w, txt.ctypes.data, txt.shape[0],
                                          schedule.ctypes.data, steps, tr.ctypes.data if trace else None, None)
        if not p:
            raise FluxHipError(f"sample_heun: {L.flux_hip_last_error().decode()}")
        out = _take_host(p, (self.cfg.channels, h, w))
        return (out, tr) if trace else out

    def sample_ancestral(self, z, h, w, txt, schedule, eta, seed=None, trace=False):
        """Euler with noise injection; `seed` (if given) seeds the host generator first."""
        z, txt, schedule = _f32(z), _f32(txt), _f32(schedule)
        steps = len(schedule) - 1
        n = self.cfg.channels * h * w
        tr = np.zeros((steps, n), np.float32) if trace else None
        L = lib()
        if seed is not None:
            L.flux_rng_seed(seed)
        p = L.flux_hip_sample_ancestral_traced(self.h, z.ctypes.data, self.cfg.channels, h, w, txt.ctypes.data,
                                               txt.shape[0], schedule.ctypes.data, steps, eta,
                                               tr.ctypes.data if trace else None, None)
        if not p:
            raise FluxHipError(f"sample_ancestral: {L.flux_hip_last_error().decode()}")
        out = _take_host(p, (self.cfg.channels, h, w))
        return (out, tr) if trace else out


class Session:
    """A device-resident sampling run: begin uploads everything, step() only queues kernels."""

    def __init__(self, model, z, h, w, txt, schedule, refs=None, txt_uncond=None, guidance=0.0):
        z, txt, schedule = _f32(z), _f32(txt), _f32(schedule)
        self.model, self.h, self.w = model, h, w
        self.steps = len(schedule) - 1
        arr, nr, keep = _refs_array(refs)
        tu = _f32(txt_uncond) if txt_uncond is not None else None
        L = lib()
        self.s = L.flux_hip_session_begin(model.h, z.ctypes.data, model.cfg.channels, h, w, arr, nr,
                                          txt.ctypes.data, txt.shape[0],
                                          tu.ctypes.data if tu is not None else None,
                                          tu.shape[0] if tu is not None else 0, guidance,
                                          schedule.ctypes.data, self.steps)
        if not self.s:
            raise FluxHipError(f"session_begin: {L.flux_hip_last_error().decode()}")

    def step(self, i):
        check(lib().flux_hip_session_step(self.s, i, None), "session_step")

    def latent(self):
        out = np.empty((self.model.cfg.channels, self.h, self.w), np.float32)
        check(lib().flux_hip_session_read_latent(self.s, out.ctypes.data), "session_read_latent")
        return out

    def close(self):
        if getattr(self, "s", None):
            lib().flux_hip_session_free(self.s)
            self.s = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def stage_timing():
    """Device milliseconds of the last collected run: (double, single, final, total)."""
    L = lib()
    return tuple(ctypes.c_double.in_dll(L, "flux_timing_transformer_" + n).value
                 for n in ("double", "single", "final", "total"))


def init_noise(channels, h, w, seed):
    p = lib().flux_init_noise(1, channels, h, w, seed)
    return _take_host(p, (channels, h, w))


def schedule(kind, n, arg=None, arg2=None):
    L = lib()
    if kind == "linear":
        p = L.flux_linear_schedule(n)
    elif kind == "power":
        p = L.flux_power_schedule(n, arg)
    elif kind == "sigmoid":
        p = L.flux_sigmoid_schedule(n, arg)
    elif kind == "resolution":
        p = L.flux_resolution_schedule(n, arg, arg2)
    elif kind == "official":
        p = L.flux_official_schedule(n, arg)
    else:
        raise ValueError(f"unknown schedule {kind!r}")
    return _take_host(p, (n + 1,))


def randn(n, seed=None):
    """n normals from the library's host generator (seeded first when `seed` is given)."""
    if seed is not None:
        lib().flux_rng_seed(seed)
    out = np.empty(n, np.float32)
    lib().flux_randn(out.ctypes.data, n)
    return out


class Vae:
    """The VAE (decoder and encoder) on the GPU, built from named tensors (uint16 = bf16, float32) or a safetensors file."""

    def __init__(self, weights=None, path=None):
        init()
        L = lib()
        if path is not None:
            self.h = L.flux_hip_vae_load_file(os.fsencode(path))
            if not self.h:
                raise FluxHipError(f"vae load_file: {L.flux_hip_last_error().decode()}")
            return
        self.h = L.flux_hip_vae_new()
        if not self.h:
            raise FluxHipError(f"vae_new: {L.flux_hip_last_error().decode()}")
        for name, a in (weights or {}).items():
            a = np.ascontiguousarray(a)
            dt = {np.dtype(np.float32): 0, np.dtype(np.float16): 1, np.dtype(np.uint16): 2}[a.dtype]
            check(L.flux_hip_vae_set_tensor(self.h, name.encode(), dt, a.ctypes.data, a.size), f"vae set_tensor({name})")

    def close(self):
        if getattr(self, "h", None):
            lib().flux_hip_vae_free(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def decode(self, latent, h, w):
        """latent [128, h, w] -> (float image [3, 16h, 16w], uint8 image [16h, 16w, 3])."""
        latent = _f32(latent)
        assert latent.size == 128 * h * w
        f = np.empty((3, 16 * h, 16 * w), np.float32)
        u = np.empty((16 * h, 16 * w, 3), np.uint8)
        check(lib().flux_hip_vae_decode(self.h, latent.ctypes.data, h, w, u.ctypes.data, f.ctypes.data), "flux_hip_vae_decode")
        return f, u

    def encode(self, img):
        """img [3, H, W] in [-1, 1], H and W multiples of 16 -> normalised latent [128, H/16, W/16]."""
        img = _f32(img)
        assert img.ndim == 3 and img.shape[0] == 3
        H, W = img.shape[1], img.shape[2]
        lat = np.empty((128, max(H // 16, 1), max(W // 16, 1)), np.float32)
        check(lib().flux_hip_vae_encode(self.h, img.ctypes.data, H, W, lat.ctypes.data), "flux_hip_vae_encode")
        return lat


class Qwen3:
    """The Qwen3 text encoder on the GPU, from named tensors (uint16 = bf16 or float32) or a model directory."""

    def __init__(self, cfg=None, weights=None, path=None):
        init()
        L = lib()
        if path is not None:
            self.h = L.flux_hip_qwen3_load_dir(os.fsencode(path))
            if not self.h:
                raise FluxHipError(f"qwen3 load_dir: {L.flux_hip_last_error().decode()}")
            return
        c = _QwenCfg(cfg.hidden, cfg.intermediate, cfg.heads, cfg.kv_heads, cfg.head_dim, cfg.layers, cfg.vocab,
                     (c_i * 3)(*cfg.out_layers), cfg.rope_theta, cfg.eps)
        self.hidden = cfg.hidden
        self.h = L.flux_hip_qwen3_new(ctypes.byref(c))
        if not self.h:
            raise FluxHipError(f"qwen3_new: {L.flux_hip_last_error().decode()}")
        for name, a in (weights or {}).items():
            self.set_tensor(name, a)

    def set_tensor(self, name, a):
        a = np.ascontiguousarray(a)
        dt = {np.dtype(np.float32): 0, np.dtype(np.float16): 1, np.dtype(np.uint16): 2}[a.dtype]
        check(lib().flux_hip_qwen3_set_tensor(self.h, name.encode(), dt, a.ctypes.data, a.size), f"qwen3 set_tensor({name})")

    def close(self):
        if getattr(self, "h", None):
            lib().flux_hip_qwen3_free(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def forward(self, ids, mask=None, hidden=None):
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        m = None if mask is None else np.ascontiguousarray(mask, dtype=np.int32)
        p = lib().flux_hip_qwen3_forward(self.h, ids.ctypes.data, None if m is None else m.ctypes.data, ids.size)
        if not p:
            raise FluxHipError(f"flux_hip_qwen3_forward: {lib().flux_hip_last_error().decode()}")
        return _take_host(p, (ids.size, 3 * (hidden or self.hidden)))
