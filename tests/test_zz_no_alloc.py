"""flux_hip_linear_static, the entry point that allocates nothing (its K slices' partial sums live in a
static device array), against flux_hip_linear on the same operands, through the C ABI: two calls in a row, the
second with a smaller input, so that what the first left in the shared array would show; a call too large to keep
K slices in the array (it runs without slices); the error for a demanded number of slices beyond the array; and the
device's free memory, which must not move across the calls."""
import ctypes

import numpy as np
import pytest

from metrics import rel_l2
from model_spec import normal_f32, f32_to_bf16, bf16_to_f32

pytestmark = pytest.mark.gpu

STATIC_BYTES = 64 << 20            # FLUX_HIP_LINEAR_STATIC_BYTES
MAX_OUTPUTS = STATIC_BYTES // 8    # FLUX_HIP_LINEAR_STATIC_MAX_OUTPUTS


def q(x):
    return bf16_to_f32(f32_to_bf16(x))


def free_bytes():
    hip_rt = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert hip_rt.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def static_linear(hip, epi, parts, N, K, lda, ldw, ldc, r0=0, r1=0):
    L = hip.lib()
    L.flux_hip_linear_static.argtypes = L.flux_hip_linear.argtypes
    arr = (hip._Part * len(parts))()
    for i, (A, W, C, g, M) in enumerate(parts):
        arr[i] = hip._Part(A, W, C, g, M)
    hip.check(L.flux_hip_linear_static(epi, len(parts), arr, N, K, lda, ldw, ldc, r0, r1), "flux_hip_linear_static")


def test_static_workspace_entry_point(oracle_mod):
    import fluxhip as hip
    hip.init()
    N, K = 3072, 12288                      # the fused output projection of a single-stream block
    W = q(normal_f32((N, K), 51, 1, 0.0, 0.02))
    gate = normal_f32((N,), 51, 2)
    dW, dg = hip.DevBuf.from_array(f32_to_bf16(W)), hip.DevBuf.from_array(gate)
    Wsw = q(normal_f32((2 * 1536, 3072), 51, 3, 0.0, 0.05))
    dWsw = hip.DevBuf.from_array(f32_to_bf16(Wsw))
    # first call: 80 rows in two parts (64 + 16); second call, right after it: 24 rows
    for rows in ((64, 16), (24,)):
        M = sum(rows)
        a = q(normal_f32((M, K), 52, M))
        res = normal_f32((M, N), 53, M)
        da = hip.DevBuf.from_array(f32_to_bf16(a))
        want = res + gate[None, :] * oracle_mod.linear(a, W)
        outs = []
        for which in ("static", "malloc"):
            dres = hip.DevBuf.from_array(res)
            parts, r = [], 0
            for m in rows:
                parts.append((da.at(r * K * 2), dW.ptr, dres.at(r * N * 4), dg.ptr, m))
                r += m
            if which == "static":
                # (a first launch of a kernel may make the runtime load code or set up its own per-queue memory:
                # the measured call is the second one with these shapes)
                warm = hip.DevBuf.from_array(res)
                static_linear(hip, hip.EPI_RESID, [(A, Wp, warm.at(C - dres.ptr), g, m) for A, Wp, C, g, m in parts], N, K, K, K, N)
                hip.sync()
                before = free_bytes()
                static_linear(hip, hip.EPI_RESID, parts, N, K, K, K, N)
                hip.sync()
                assert free_bytes() == before          # nothing was allocated (or freed) on the device
            else:
                hip.linear(hip.EPI_RESID, parts, N, K, K, K, N)
            outs.append(dres.to_array(np.float32, (M, N)))
        assert rel_l2(outs[0], want) < 2e-6, rows
        assert rel_l2(outs[0], outs[1]) < 2e-6, rows   # fp32 results: the same up to the order of the slices' sums
        # the bf16 and SiLU(gate) * up second passes read the same array
        x = q(normal_f32((M, 3072), 54, M))
        dx = hip.DevBuf.from_array(f32_to_bf16(x))
        lin = oracle_mod.linear(x, Wsw)
        want_sw = oracle_mod.silu(lin[:, :1536]) * lin[:, 1536:]
        got = {}
        for which in ("static", "malloc"):
            o = hip.DevBuf(M * 1536 * 2)
            p = [(dx.ptr, dWsw.ptr, o.ptr, None, M)]
            (static_linear if which == "static" else lambda h, *a: h.linear(*a))(hip, hip.EPI_SWIGLU, p, 2 * 1536, 3072, 3072, 3072, 1536, 0, 1536)
            got[which] = bf16_to_f32(o.to_array(np.uint16, (M, 1536)))
        assert rel_l2(got["static"], want_sw) < 4e-3
        assert rel_l2(got["static"], got["malloc"]) < 2e-3
    # a shape that does not split at all runs as well (no workspace touched) ...
    M = 300
    a = q(normal_f32((M, 256), 55, 1))
    W2 = q(normal_f32((256, 256), 55, 2, 0.0, 0.1))
    da, dW2, o = hip.DevBuf.from_array(f32_to_bf16(a)), hip.DevBuf.from_array(f32_to_bf16(W2)), hip.DevBuf(M * 256 * 4)
    static_linear(hip, hip.EPI_F32, [(da.ptr, dW2.ptr, o.ptr, None, M)], 256, 256, 256, 256, 256)
    assert rel_l2(o.to_array(np.float32, (M, 256)), oracle_mod.linear(a, W2)) < 2e-6
    # ... and so does one whose outputs exceed what two slices of partial sums could keep in the array: as one launch
    # without slices, bit for bit what flux_hip_linear gives with its K slices switched off, and nothing allocated
    big_rows = MAX_OUTPUTS // N + 1
    ab = q(normal_f32((big_rows, K), 56, 1))
    dab = hip.DevBuf.from_array(f32_to_bf16(ab))
    o1, o2 = hip.DevBuf(big_rows * N * 4), hip.DevBuf(big_rows * N * 4)
    static_linear(hip, hip.EPI_F32, [(dab.ptr, dW.ptr, o1.ptr, None, big_rows)], N, K, K, K, N)
    hip.sync()
    before = free_bytes()
    static_linear(hip, hip.EPI_F32, [(dab.ptr, dW.ptr, o1.ptr, None, big_rows)], N, K, K, K, N)
    hip.sync()
    assert free_bytes() == before
    L = hip.lib()
    L.flux_hip_linear_enable_splitk(0)
    try:
        hip.linear(hip.EPI_F32, [(dab.ptr, dW.ptr, o2.ptr, None, big_rows)], N, K, K, K, N)
    finally:
        L.flux_hip_linear_enable_splitk(1)
    np.testing.assert_array_equal(o1.to_array(np.float32, (big_rows, N)), o2.to_array(np.float32, (big_rows, N)))
    # a demanded number of slices beyond the array is the one request it refuses, with a reason, before anything is launched
    L.flux_hip_linear_force_split(4)
    try:
        with pytest.raises(hip.FluxHipError) as err:
            static_linear(hip, hip.EPI_F32, [(dab.ptr, dW.ptr, o1.ptr, None, big_rows)], N, K, K, K, N)
        assert "beyond the maximum" in str(err.value)
        # ... while the same demand on a size that fits is served
        static_linear(hip, hip.EPI_F32, [(dab.ptr, dW.ptr, o2.ptr, None, 64)], N, K, K, K, N)
        assert rel_l2(o2.to_array(np.float32, (big_rows, N))[:64], oracle_mod.linear(ab[:64], W)) < 2e-6
    finally:
        L.flux_hip_linear_force_split(0)
