"""Parity of every HIP operator against the CPU oracle, through the C ABI (include/flux_hip.h).

Inputs are rounded to bf16 first, so both sides see identical values; what remains is fp32
accumulation order and the bf16 rounding of outputs. Tolerances are stated per test.
"""
import numpy as np
import pytest

from metrics import rel_l2
from model_spec import normal_f32, f32_to_bf16, bf16_to_f32

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    import fluxhip
    fluxhip.init()
    yield fluxhip
    fluxhip.lib().flux_hip_linear_force_tile(-1)


def q(x):
    """Round to bf16 and come back: the values a bf16 tensor actually holds."""
    return bf16_to_f32(f32_to_bf16(x))


def dev_bf16(hip, x):
    return hip.DevBuf.from_array(f32_to_bf16(x))


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4, 5, 6, 7])
@pytest.mark.parametrize("M", [1, 37, 130, 300])
def test_linear_bf16_and_f32(hip, oracle_mod, tile, M):
    N, K = (768 if tile >= 5 else 512), 192        # the 192-wide tiles need N % 192 == 0
    hip.lib().flux_hip_linear_force_tile(tile)
    x = q(normal_f32((M, K), 3, 1))
    W = q(normal_f32((N + 64, K), 3, 2, 0.0, 0.1))
    want = oracle_mod.linear(x, W[64:64 + N])
    dx, dW = dev_bf16(hip, x), dev_bf16(hip, W)
    # bf16 output, weight rows start at 64
    out = hip.DevBuf(M * N * 2)
    hip.linear(hip.EPI_BF16, [(dx.ptr, dW.ptr, out.ptr, None, M)], N, K, K, K, N, 64, 0)
    got = bf16_to_f32(out.to_array(np.uint16, (M, N)))
    assert rel_l2(got, want) < 4e-3          # bf16 output rounding: 2^-9 relative per element
    # fp32 output is accumulation-order noise only
    out32 = hip.DevBuf(M * N * 4)
    hip.linear(hip.EPI_F32, [(dx.ptr, dW.ptr, out32.ptr, None, M)], N, K, K, K, N, 64, 0)
    assert rel_l2(out32.to_array(np.float32, (M, N)), want) < 2e-6
    # transposed fp32 output
    outT = hip.DevBuf(M * N * 4)
    hip.linear(hip.EPI_F32_T, [(dx.ptr, dW.ptr, outT.ptr, None, M)], N, K, K, K, M, 64, 0)
    assert rel_l2(outT.to_array(np.float32, (N, M)).T, want) < 2e-6


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4, 5, 6, 7])
def test_linear_two_parts_resid_and_strides(hip, oracle_mod, tile):
    """Two row ranges with different weights, strided A (lda > K), gated residual epilogue."""
    hip.lib().flux_hip_linear_force_tile(tile)
    M0, M1, N, K, lda = 70, 200, (768 if tile >= 5 else 256), 128, 320
    a = q(normal_f32((M0 + M1, lda), 4, 1))
    W0 = q(normal_f32((N, K), 4, 2, 0.0, 0.1))
    W1 = q(normal_f32((N, K), 4, 3, 0.0, 0.1))
    res = normal_f32((M0 + M1, N), 4, 4)
    g0 = normal_f32((N,), 4, 5)
    g1 = normal_f32((N,), 4, 6)
    col = 64  # A starts at column 64 of the strided buffer
    want = res.copy()
    want[:M0] += g0 * oracle_mod.linear(a[:M0, col:col + K], W0)
    want[M0:] += g1 * oracle_mod.linear(a[M0:, col:col + K], W1)
    da, dW0, dW1 = dev_bf16(hip, a), dev_bf16(hip, W0), dev_bf16(hip, W1)
    dres = hip.DevBuf.from_array(res)
    dg0, dg1 = hip.DevBuf.from_array(g0), hip.DevBuf.from_array(g1)
    hip.linear(hip.EPI_RESID, [(da.at(col * 2), dW0.ptr, dres.ptr, dg0.ptr, M0),
                               (da.at((M0 * lda + col) * 2), dW1.ptr, dres.at(M0 * N * 4), dg1.ptr, M1)],
               N, K, lda, K, N)
    assert rel_l2(dres.to_array(np.float32, (M0 + M1, N)), want) < 2e-6


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4, 5, 6, 7])
def test_linear_swiglu(hip, oracle_mod, tile):
    """silu(x Wg^T) * (x Wu^T) with gate/up rows at arbitrary offsets and a strided output."""
    hip.lib().flux_hip_linear_force_tile(tile)
    M, K, mlp, ldc, r0 = 150, 128, 384, 512, 128
    x = q(normal_f32((M, K), 5, 1))
    W = q(normal_f32((r0 + 2 * mlp, K), 5, 2, 0.0, 0.15))
    g = oracle_mod.linear(x, W[r0:r0 + mlp])
    u = oracle_mod.linear(x, W[r0 + mlp:])
    want = oracle_mod.silu(g) * u
    dx, dW = dev_bf16(hip, x), dev_bf16(hip, W)
    out = hip.DevBuf.from_array(np.zeros((M, ldc), np.uint16))
    hip.linear(hip.EPI_SWIGLU, [(dx.ptr, dW.ptr, out.at(64 * 2), None, M)], 2 * mlp, K, K, K, ldc, r0, r0 + mlp)
    got = bf16_to_f32(out.to_array(np.uint16, (M, ldc)))
    assert rel_l2(got[:, 64:64 + mlp], want) < 4e-3
    assert not got[:, :64].any() and not got[:, 64 + mlp:].any()   # nothing written outside


@pytest.mark.parametrize("N", [640, 768, 896, 1152])
@pytest.mark.parametrize("K", [256, 448])
def test_linear_tile_with_cut_last_column_tile(hip, oracle_mod, N, K):
    """256 x 224 (tile 11) divides none of these widths: the last column tile ends after 192, 96, 224 and 32 columns (in
    the second wave's columns, inside the first wave's, nowhere, inside the first pair of blocks). Gated residual
    epilogue on two row ranges, and the bf16 store where its pairs of 16-column blocks allow the cut (not at 640):
    against the oracle, and bit for bit against the 128 x 128 tile, which accumulates in the same order."""
    L = hip.lib()
    M0, M1 = 300, 70
    a = q(normal_f32((M0 + M1, K), 41, 1))
    W0 = q(normal_f32((N, K), 41, 2, 0.0, 0.1))
    W1 = q(normal_f32((N, K), 41, 3, 0.0, 0.1))
    res = normal_f32((M0 + M1, N), 41, 4)
    g0, g1 = normal_f32((N,), 41, 5), normal_f32((N,), 41, 6)
    want = res.copy()
    want[:M0] += g0 * oracle_mod.linear(a[:M0], W0)
    want[M0:] += g1 * oracle_mod.linear(a[M0:], W1)
    da, dW0, dW1 = dev_bf16(hip, a), dev_bf16(hip, W0), dev_bf16(hip, W1)
    dg0, dg1 = hip.DevBuf.from_array(g0), hip.DevBuf.from_array(g1)
    got = {}
    for tile in (11, 1):
        L.flux_hip_linear_force_tile(tile)
        L.flux_hip_linear_probe(hip.EPI_RESID)
        # (a guard row behind the output: nothing may be written past the last column)
        dres = hip.DevBuf.from_array(np.concatenate([res, np.full((1, N), 7.0, np.float32)]))
        hip.linear(hip.EPI_RESID, [(da.ptr, dW0.ptr, dres.ptr, dg0.ptr, M0), (da.at(M0 * K * 2), dW1.ptr, dres.at(M0 * N * 4), dg1.ptr, M1)],
                   N, K, K, K, N)
        tiles = np.zeros(4, np.int32)
        assert L.flux_hip_linear_probe_read_launches(4, tiles.ctypes.data, None) == 1 and tiles[0] == tile
        full = dres.to_array(np.float32, (M0 + M1 + 1, N))
        assert (full[-1] == 7.0).all()
        got[tile] = full[:-1]
    assert rel_l2(got[11], want) < 2e-6
    assert np.array_equal(got[11], got[1])
    # bf16 output with a row stride wider than N: the columns behind N stay as they were
    ldc = N + 64
    x = a[:M0]
    want16 = oracle_mod.linear(x, W0)
    out = {}
    for tile in (11, 1):
        L.flux_hip_linear_force_tile(tile)
        L.flux_hip_linear_probe(hip.EPI_BF16)
        dout = hip.DevBuf.from_array(np.full((M0, ldc), 0x4242, np.uint16))
        hip.linear(hip.EPI_BF16, [(da.ptr, dW0.ptr, dout.ptr, None, M0)], N, K, K, K, ldc, 0, 0)
        tiles = np.zeros(4, np.int32)
        assert L.flux_hip_linear_probe_read_launches(4, tiles.ctypes.data, None) == 1
        assert tiles[0] == (tile if tile == 1 or (N % 224) % 112 % 32 == 0 else 1)   # refused where a pair would be cut in two
        out[tile] = dout.to_array(np.uint16, (M0, ldc))
        assert (out[tile][:, N:] == 0x4242).all()
    assert np.array_equal(out[11], out[1])
    assert rel_l2(bf16_to_f32(out[11][:, :N]), want16) < 4e-3
    L.flux_hip_linear_probe(-1)
    L.flux_hip_linear_force_tile(-1)


@pytest.mark.parametrize("epi,N", [("resid", 3072), ("bf16", 9216)])
def test_linear_cut_tile_at_the_double_stream_shapes(hip, epi, N):
    """256 x 224 where the model uses it: 4096 image + 512 text rows with weights of their own, K = 3072, the gated residual
    add at N = 3072 (252 tiles: one per workgroup, the last of every 14 cut off after 160 columns) and the bf16 store at
    N = 9216 (756 tiles: three per workgroup in one pipeline, a cut tile of 32 columns in the middle of some workgroups'
    runs, so the first barrier of the tile behind it must not count on stores that were never issued). Bit for bit what
    the 256 x 256 tile gives, which the whole-model tests hold against the oracle; nothing written behind the outputs."""
    L = hip.lib()
    K, M0, M1 = 3072, 4096, 512
    a = q(normal_f32((M0 + M1, K), 43, 1))
    W0 = q(normal_f32((N, K), 43, 2, 0.0, 0.02))
    W1 = q(normal_f32((N, K), 43, 3, 0.0, 0.02))
    da, dW0, dW1 = dev_bf16(hip, a), dev_bf16(hip, W0), dev_bf16(hip, W1)
    got = {}
    for tile in (11, 2):
        L.flux_hip_linear_force_tile(tile)
        L.flux_hip_linear_probe(hip.EPI_RESID if epi == "resid" else hip.EPI_BF16)
        if epi == "resid":
            res = normal_f32((M0 + M1 + 1, N), 43, 4)
            g0, g1 = hip.DevBuf.from_array(normal_f32((N,), 43, 5)), hip.DevBuf.from_array(normal_f32((N,), 43, 6))
            out = hip.DevBuf.from_array(res)
            hip.linear(hip.EPI_RESID, [(da.ptr, dW0.ptr, out.ptr, g0.ptr, M0), (da.at(M0 * K * 2), dW1.ptr, out.at(M0 * N * 4), g1.ptr, M1)],
                       N, K, K, K, N)
            full = out.to_array(np.float32, (M0 + M1 + 1, N))
            assert np.array_equal(full[-1], res[-1])
        else:
            out = hip.DevBuf.from_array(np.full((M0 + M1 + 1, N), 0x4242, np.uint16))
            hip.linear(hip.EPI_BF16, [(da.ptr, dW0.ptr, out.ptr, None, M0), (da.at(M0 * K * 2), dW1.ptr, out.at(M0 * N * 2), None, M1)],
                       N, K, K, K, N, 0, 0)
            full = out.to_array(np.uint16, (M0 + M1 + 1, N))
            assert (full[-1] == 0x4242).all()
        tiles = np.zeros(4, np.int32)
        assert L.flux_hip_linear_probe_read_launches(4, tiles.ctypes.data, None) == 1 and tiles[0] == tile
        got[tile] = full[:-1]
    L.flux_hip_linear_probe(-1)
    L.flux_hip_linear_force_tile(-1)
    assert np.array_equal(got[11], got[2])
    assert np.isfinite(got[11].astype(np.float32)).all() if epi == "resid" else True


@pytest.mark.parametrize("tile", [2, 5, 6, 7])
@pytest.mark.parametrize("K", [64, 128, 192, 256, 448])
def test_linear_large_tile_k_steps(hip, oracle_mod, K, tile):
    """The hand-pipelined loop of the 4-wave tiles peels its last two K steps: every count from one
    step up, with a ragged row count and several tiles in both directions."""
    hip.lib().flux_hip_linear_force_tile(tile)
    M, N = 300, 768
    x = q(normal_f32((M, K), 31, 1))
    W = q(normal_f32((N, K), 31, 2, 0.0, 0.1))
    want = oracle_mod.linear(x, W)
    dx, dW = dev_bf16(hip, x), dev_bf16(hip, W)
    out32 = hip.DevBuf(M * N * 4)
    hip.linear(hip.EPI_F32, [(dx.ptr, dW.ptr, out32.ptr, None, M)], N, K, K, K, N, 0, 0)
    assert rel_l2(out32.to_array(np.float32, (M, N)), want) < 2e-6
    hip.lib().flux_hip_linear_force_tile(-1)


@pytest.mark.parametrize("tile", [2, 5, 6, 7])
def test_linear_workgroups_walk_several_tiles(hip, oracle_mod, tile):
    """More tiles than compute units: a workgroup of the 4-wave kernel goes on to further tiles (and requests the
    next tile's first stage before it stores the finished one). Ragged row counts, two row ranges, every epilogue
    of the transformer; the result must also be bit for bit what one workgroup per tile gives."""
    L = hip.lib()
    L.flux_hip_linear_force_tile(tile)
    K, N = 192, 6144
    Ms = (1500, 1200)
    xs = [q(normal_f32((M, K), 41, 1 + i)) for i, M in enumerate(Ms)]
    W = q(normal_f32((N, K), 41, 5, 0.0, 0.1))
    gate = normal_f32((N,), 41, 6)
    res0 = [normal_f32((M, N), 41, 7 + i) for i, M in enumerate(Ms)]
    dxs, dW, dg = [dev_bf16(hip, x) for x in xs], dev_bf16(hip, W), hip.DevBuf.from_array(gate)
    outs = {}
    for persistent in (1, 0):
        L.flux_hip_linear_persistent(persistent)
        # bf16 store
        ob = [hip.DevBuf(M * N * 2) for M in Ms]
        hip.linear(hip.EPI_BF16, [(dx.ptr, dW.ptr, o.ptr, None, M) for dx, o, M in zip(dxs, ob, Ms)], N, K, K, K, N, 0, 0)
        # gated residual
        orr = [hip.DevBuf.from_array(r) for r in res0]
        hip.linear(hip.EPI_RESID, [(dx.ptr, dW.ptr, o.ptr, dg.ptr, M) for dx, o, M in zip(dxs, orr, Ms)], N, K, K, K, N, 0, 0)
        # silu(gate) * up with the gate rows in the first half of W and the up rows in the second
        osw = [hip.DevBuf(M * (N // 2) * 2) for M in Ms]
        hip.linear(hip.EPI_SWIGLU, [(dx.ptr, dW.ptr, o.ptr, None, M) for dx, o, M in zip(dxs, osw, Ms)], N, K, K, K, N // 2, 0, N // 2)
        outs[persistent] = ([o.to_array(np.uint16, (M, N)) for o, M in zip(ob, Ms)],
                            [o.to_array(np.float32, (M, N)) for o, M in zip(orr, Ms)],
                            [o.to_array(np.uint16, (M, N // 2)) for o, M in zip(osw, Ms)])
    L.flux_hip_linear_persistent(1)
    L.flux_hip_linear_force_tile(-1)
    for i, (x, M) in enumerate(zip(xs, Ms)):
        want = oracle_mod.linear(x, W)
        assert rel_l2(bf16_to_f32(outs[1][0][i]), want) < 4e-3
        assert rel_l2(outs[1][1][i], res0[i] + gate[None, :] * want) < 2e-6
        assert rel_l2(bf16_to_f32(outs[1][2][i]), oracle_mod.silu(want[:, :N // 2]) * want[:, N // 2:]) < 4e-3
        for k in range(3):
            assert np.array_equal(outs[1][k][i], outs[0][k][i])


@pytest.mark.parametrize("tile", [-1, 0, 1, 6])
def test_linear_split_k_other_epilogues(hip, oracle_mod, tile):
    """Few rows, long K: the bf16, fp32 and SwiGLU epilogues also run as K slices plus a finishing pass
    (SwiGLU only when gate and up rows are adjacent). Same answer with the split switched off."""
    hip.lib().flux_hip_linear_force_tile(tile)
    M, K, mlp, r0 = 80, 3072, 384, 64
    x = q(normal_f32((M, K), 33, 1))
    W = q(normal_f32((r0 + 2 * mlp, K), 33, 2, 0.0, 0.05))
    lin = oracle_mod.linear(x, W[r0:])
    want_sw = oracle_mod.silu(lin[:, :mlp]) * lin[:, mlp:]
    dx, dW = dev_bf16(hip, x), dev_bf16(hip, W)
    res = {}
    for on in (1, 0):
        hip.lib().flux_hip_linear_enable_splitk(on)
        o_bf = hip.DevBuf(M * 2 * mlp * 2)
        hip.linear(hip.EPI_BF16, [(dx.ptr, dW.ptr, o_bf.ptr, None, M)], 2 * mlp, K, K, K, 2 * mlp, r0, 0)
        o_f = hip.DevBuf(M * 2 * mlp * 4)
        hip.linear(hip.EPI_F32, [(dx.ptr, dW.ptr, o_f.ptr, None, M)], 2 * mlp, K, K, K, 2 * mlp, r0, 0)
        o_sw = hip.DevBuf(M * mlp * 2)
        hip.linear(hip.EPI_SWIGLU, [(dx.ptr, dW.ptr, o_sw.ptr, None, M)], 2 * mlp, K, K, K, mlp, r0, r0 + mlp)
        res[on] = (bf16_to_f32(o_bf.to_array(np.uint16, (M, 2 * mlp))), o_f.to_array(np.float32, (M, 2 * mlp)),
                   bf16_to_f32(o_sw.to_array(np.uint16, (M, mlp))))
    hip.lib().flux_hip_linear_enable_splitk(1)
    for on in (1, 0):
        assert rel_l2(res[on][0], lin) < 4e-3
        assert rel_l2(res[on][1], lin) < 2e-6
        assert rel_l2(res[on][2], want_sw) < 4e-3
    # gate and up rows not adjacent: must still be right (no split possible)
    o_sw = hip.DevBuf(M * 128 * 2)
    hip.linear(hip.EPI_SWIGLU, [(dx.ptr, dW.ptr, o_sw.ptr, None, M)], 256, K, K, K, 128, r0, r0 + 2 * mlp - 128)
    want = oracle_mod.silu(lin[:, :128]) * lin[:, 2 * mlp - 128:]
    assert rel_l2(bf16_to_f32(o_sw.to_array(np.uint16, (M, 128))), want) < 4e-3


@pytest.mark.parametrize("tile", [-1, 0, 2, 3, 5, 6, 7])
def test_linear_split_k(hip, oracle_mod, tile):
    """Long K, few output tiles: the residual epilogue splits K over workgroups (two passes through a
    workspace, fixed summation order). Two row ranges, repeated runs must agree bit for bit."""
    hip.lib().flux_hip_linear_force_tile(tile)
    M0, M1, N, K = 64, 16, (768 if tile >= 5 else 256), 4096
    a = q(normal_f32((M0 + M1, K), 20, 1))
    W0 = q(normal_f32((N, K), 20, 2, 0.0, 0.05))
    W1 = q(normal_f32((N, K), 20, 3, 0.0, 0.05))
    res = normal_f32((M0 + M1, N), 20, 4)
    g0, g1 = normal_f32((N,), 20, 5), normal_f32((N,), 20, 6)
    want = res.copy()
    want[:M0] += g0 * oracle_mod.linear(a[:M0], W0)
    want[M0:] += g1 * oracle_mod.linear(a[M0:], W1)
    da, dW0, dW1 = dev_bf16(hip, a), dev_bf16(hip, W0), dev_bf16(hip, W1)
    dg0, dg1 = hip.DevBuf.from_array(g0), hip.DevBuf.from_array(g1)
    outs = []
    for on in (1, 1, 0):
        hip.lib().flux_hip_linear_enable_splitk(on)
        dres = hip.DevBuf.from_array(res)
        hip.linear(hip.EPI_RESID, [(da.ptr, dW0.ptr, dres.ptr, dg0.ptr, M0),
                                   (da.at(M0 * K * 2), dW1.ptr, dres.at(M0 * N * 4), dg1.ptr, M1)], N, K, K, K, N)
        outs.append(dres.to_array(np.float32, (M0 + M1, N)))
    hip.lib().flux_hip_linear_enable_splitk(1)
    assert np.array_equal(outs[0], outs[1])            # deterministic
    for o in outs:
        assert rel_l2(o, want) < 2e-6
    # one-part, ragged K slices (K/64 = 25 steps does not divide evenly)
    K2 = 1600
    x = q(normal_f32((40, K2), 20, 7))
    W = q(normal_f32((128, K2), 20, 8, 0.0, 0.05))
    r = normal_f32((40, 128), 20, 9)
    dres = hip.DevBuf.from_array(r)
    dx, dW = dev_bf16(hip, x), dev_bf16(hip, W)
    hip.linear(hip.EPI_RESID, [(dx.ptr, dW.ptr, dres.ptr, dg0.ptr, 40)], 128, K2, K2, K2, 128)
    assert rel_l2(dres.to_array(np.float32, (40, 128)), r + g0[:128] * oracle_mod.linear(x, W)) < 2e-6


@pytest.mark.parametrize("tile", [-1, 1, 6])
@pytest.mark.parametrize("shape", [(64, 16, 768, 4096), (80, 0, 3072, 12288), (300, 212, 256, 256)])
def test_linear_residual_then_adaln(hip, oracle_mod, shape, tile):
    """A residual projection that runs as K slices also writes the AdaLN of the rows it updated; x is then
    bit for bit what the plain two-pass form gives, the normalised rows agree with the stand-alone kernel
    and with the oracle. A projection that does not split reports that it left the normalisation to the caller."""
    M0, M1, N, K = shape
    hip.lib().flux_hip_linear_force_tile(tile)             # a forced tile that does not divide N is ignored
    a = q(normal_f32((M0 + M1, K), 24, 1))
    W0, W1 = q(normal_f32((N, K), 24, 2, 0.0, 0.05)), q(normal_f32((N, K), 24, 3, 0.0, 0.05))
    res = normal_f32((M0 + M1, N), 24, 4)
    g0, g1 = normal_f32((N,), 24, 5), normal_f32((N,), 24, 6)
    sh = [normal_f32((N,), 24, 7 + i, 0.0, 0.3) for i in range(2)]
    sc = [normal_f32((N,), 24, 9 + i, 0.0, 0.3) for i in range(2)]
    da, dW0, dW1 = dev_bf16(hip, a), dev_bf16(hip, W0), dev_bf16(hip, W1)
    dg0, dg1 = hip.DevBuf.from_array(g0), hip.DevBuf.from_array(g1)
    dsh, dsc = [hip.DevBuf.from_array(v) for v in sh], [hip.DevBuf.from_array(v) for v in sc]
    parts = lambda dres: [(da.ptr, dW0.ptr, dres.ptr, dg0.ptr, M0), (da.at(M0 * K * 2), dW1.ptr, dres.at(M0 * N * 4), dg1.ptr, M1)]
    # plain: projection, then the stand-alone AdaLN kernel
    dres = hip.DevBuf.from_array(res)
    hip.linear(hip.EPI_RESID, parts(dres), N, K, K, K, N)
    x_plain = dres.to_array(np.float32, (M0 + M1, N))
    dn = hip.DevBuf((M0 + M1) * N * 2)
    hip.check(hip.lib().flux_hip_adaln_norm(dn.ptr, N, dres.ptr, M0 + M1, N, M0, dsh[0].ptr, dsc[0].ptr, dsh[1].ptr, dsc[1].ptr, 1e-6))
    n_plain = bf16_to_f32(dn.to_array(np.uint16, (M0 + M1, N)))
    # fused
    dres2 = hip.DevBuf.from_array(res)
    dn2 = hip.DevBuf.from_array(np.full((M0 + M1, N), 0x7fc0, np.uint16))
    fused = hip.linear_resid_adaln(parts(dres2), N, K, K, K, N, [(dn2.ptr, dsh[0].ptr, dsc[0].ptr), (dn2.at(M0 * N * 2), dsh[1].ptr, dsc[1].ptr)])
    x_fused = dres2.to_array(np.float32, (M0 + M1, N))
    assert fused == (K > 256)                              # K = 256 is too short to slice
    np.testing.assert_array_equal(x_fused, x_plain)
    want_x = res.copy()
    want_x[:M0] += g0 * oracle_mod.linear(a[:M0], W0)
    if M1:
        want_x[M0:] += g1 * oracle_mod.linear(a[M0:], W1)
    assert rel_l2(x_fused, want_x) < 2e-6
    if fused:
        n_fused = bf16_to_f32(dn2.to_array(np.uint16, (M0 + M1, N)))
        want_n = oracle_mod.adaln(want_x[:M0], sh[0], sc[0])
        if M1:
            want_n = np.concatenate([want_n, oracle_mod.adaln(want_x[M0:], sh[1], sc[1])])
        assert rel_l2(n_fused, want_n) < 4e-3
        assert rel_l2(n_fused, n_plain) < 2e-3 and (n_fused != n_plain).mean() < 0.02     # same values up to the order of the row sums
    # no AdaLN asked for: the plain projection, never "fused"
    dres3 = hip.DevBuf.from_array(res)
    assert hip.linear_resid_adaln(parts(dres3), N, K, K, K, N, None) is False
    np.testing.assert_array_equal(dres3.to_array(np.float32, (M0 + M1, N)), x_plain)
    hip.lib().flux_hip_linear_force_tile(-1)


def test_linear_residual_then_rms_norm(hip, oracle_mod):
    """The same second pass with the text encoder's RMS norm (no shift, scale = the norm's weight)."""
    M, N, K = 96, 2560, 4096
    a = q(normal_f32((M, K), 25, 1))
    W = q(normal_f32((N, K), 25, 2, 0.0, 0.05))
    res = normal_f32((M, N), 25, 3)
    g = np.ones(N, np.float32)
    wn = normal_f32((N,), 25, 4, 1.0, 0.2)
    da, dW, dg, dwn = dev_bf16(hip, a), dev_bf16(hip, W), hip.DevBuf.from_array(g), hip.DevBuf.from_array(wn)
    dres = hip.DevBuf.from_array(res)
    dn = hip.DevBuf.from_array(np.full((M, N), 0x7fc0, np.uint16))
    fused = hip.linear_resid_adaln([(da.ptr, dW.ptr, dres.ptr, dg.ptr, M)], N, K, K, K, N, [(dn.ptr, None, dwn.ptr)])
    assert fused
    x = dres.to_array(np.float32, (M, N))
    want_x = res + oracle_mod.linear(a, W)
    assert rel_l2(x, want_x) < 2e-6
    assert rel_l2(bf16_to_f32(dn.to_array(np.uint16, (M, N))), oracle_mod.qwen3_rms_norm(want_x, wn, 1e-6)) < 4e-3
    # shift given for one part only: rejected before anything runs
    with pytest.raises(hip.FluxHipError):
        hip.linear_resid_adaln([(da.ptr, dW.ptr, dres.ptr, dg.ptr, 64), (da.ptr, dW.ptr, dres.ptr, dg.ptr, 32)], N, K, K, K, N,
                               [(dn.ptr, None, dwn.ptr), (dn.ptr, dwn.ptr, dwn.ptr)])


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4, 5, 6, 7])
@pytest.mark.parametrize("M", [45, 700])
def test_linear_qkv_swiglu_one_launch(hip, oracle_mod, tile, M):
    """The fused projection of a single-stream block (rows [Q, K, V, gate, up], flux_transformer.c:3034-3058) as ONE
    launch: bit for bit what the two launches (bf16 store, SiLU(gate) * up) give on the same tile, and right
    against the oracle. Strided outputs; nothing written outside them."""
    import ctypes
    L = hip.lib()
    L.flux_hip_linear_qkv_swiglu.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 8
    L.flux_hip_linear_force_tile(tile)
    K, qc, mlp = 192, 768, 1536                         # both widths are multiples of every tile width (64 ... 256)
    ldq, ldm = qc + 64, mlp + 128
    x = q(normal_f32((M, K), 61, 1))
    W = q(normal_f32((qc + 2 * mlp, K), 61, 2, 0.0, 0.1))
    dx, dW = dev_bf16(hip, x), dev_bf16(hip, W)
    fq = hip.DevBuf.from_array(np.zeros((M, ldq), np.uint16))
    fm = hip.DevBuf.from_array(np.zeros((M, ldm), np.uint16))
    hip.check(L.flux_hip_linear_qkv_swiglu(dx.ptr, dW.ptr, fq.ptr, fm.at(64 * 2), M, qc, mlp, K, K, K, ldq, ldm), "flux_hip_linear_qkv_swiglu")
    tq = hip.DevBuf.from_array(np.zeros((M, ldq), np.uint16))
    tm = hip.DevBuf.from_array(np.zeros((M, ldm), np.uint16))
    L.flux_hip_linear_enable_splitk(0)
    try:
        hip.linear(hip.EPI_BF16, [(dx.ptr, dW.ptr, tq.ptr, None, M)], qc, K, K, K, ldq, 0, 0)
        hip.linear(hip.EPI_SWIGLU, [(dx.ptr, dW.ptr, tm.at(64 * 2), None, M)], 2 * mlp, K, K, K, ldm, qc, qc + mlp)
    finally:
        L.flux_hip_linear_enable_splitk(1)
        L.flux_hip_linear_force_tile(-1)
    got_q, got_m = fq.to_array(np.uint16, (M, ldq)), fm.to_array(np.uint16, (M, ldm))
    np.testing.assert_array_equal(got_q, tq.to_array(np.uint16, (M, ldq)))
    np.testing.assert_array_equal(got_m, tm.to_array(np.uint16, (M, ldm)))
    lin = oracle_mod.linear(x, W)
    assert rel_l2(bf16_to_f32(got_q[:, :qc]), lin[:, :qc]) < 4e-3
    assert rel_l2(bf16_to_f32(got_m[:, 64:64 + mlp]), oracle_mod.silu(lin[:, qc:qc + mlp]) * lin[:, qc + mlp:]) < 4e-3
    assert not got_q[:, qc:].any() and not got_m[:, :64].any() and not got_m[:, 64 + mlp:].any()


@pytest.mark.parametrize("tile,M", [(8, 1), (8, 37), (8, 64), (9, 80), (9, 128), (10, 80), (10, 96)])
@pytest.mark.parametrize("K", [64, 192, 320, 448, 1024])
def test_linear_deep_ring_tiles(hip, oracle_mod, tile, M, K):
    """Tiles 8 and 9: the 64 x 128 and 128 x 128 tiles with a ring of 6 and 5 LDS stages for parts of few rows.
    K steps from one (fewer than the ring holds) to sixteen (the ring wraps several times); bf16, fp32, gated
    residual over two parts, SwiGLU and the fused [Q|K|V|gate|up] launch; bit for bit what the two-stage form of the
    same tile gives (same MFMA order), and right against the oracle. The launch probe confirms which tile ran."""
    import ctypes
    L = hip.lib()
    L.flux_hip_linear_qkv_swiglu.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 8
    N, mlp = 512, 256
    x = q(normal_f32((M, K), 71, 1))
    x2 = q(normal_f32((M // 2 + 1, K), 71, 2))
    W = q(normal_f32((N + 2 * mlp, K), 71, 3, 0.0, 0.1))
    gate = normal_f32((N,), 71, 4)
    res = [normal_f32((M, N), 71, 5), normal_f32((M // 2 + 1, N), 71, 6)]
    dx, dx2, dW, dg = dev_bf16(hip, x), dev_bf16(hip, x2), dev_bf16(hip, W), hip.DevBuf.from_array(gate)
    outs = {}
    L.flux_hip_linear_enable_splitk(0)
    try:
        for t in (tile, 1 if tile == 10 else tile - 8):            # tile 0 = 64 x 128 and tile 1 = 128 x 128 with two stages
            L.flux_hip_linear_force_tile(t)
            L.flux_hip_linear_probe(hip.EPI_BF16)
            o16, o32 = hip.DevBuf(M * N * 2), hip.DevBuf(M * N * 4)
            hip.linear(hip.EPI_BF16, [(dx.ptr, dW.ptr, o16.ptr, None, M)], N, K, K, K, N)
            tiles, ms = np.zeros(4, np.int32), np.zeros(4, np.float32)
            assert L.flux_hip_linear_probe_read_launches(4, tiles.ctypes.data, ms.ctypes.data) == 1 and tiles[0] == t
            L.flux_hip_linear_probe(-1)
            hip.linear(hip.EPI_F32, [(dx.ptr, dW.ptr, o32.ptr, None, M)], N, K, K, K, N)
            r = [hip.DevBuf.from_array(a) for a in res]
            hip.linear(hip.EPI_RESID, [(dx.ptr, dW.ptr, r[0].ptr, dg.ptr, M), (dx2.ptr, dW.at(64 * K * 2), r[1].ptr, dg.ptr, M // 2 + 1)], N, K, K, K, N)
            sw = hip.DevBuf(M * mlp * 2)
            hip.linear(hip.EPI_SWIGLU, [(dx.ptr, dW.ptr, sw.ptr, None, M)], 2 * mlp, K, K, K, mlp, N, N + mlp)
            fq, fm = hip.DevBuf(M * N * 2), hip.DevBuf(M * mlp * 2)
            hip.check(L.flux_hip_linear_qkv_swiglu(dx.ptr, dW.ptr, fq.ptr, fm.ptr, M, N, mlp, K, K, K, N, mlp), "flux_hip_linear_qkv_swiglu")
            outs[t] = [o16.to_array(np.uint16, (M, N)), o32.to_array(np.float32, (M, N)), r[0].to_array(np.float32, (M, N)),
                       r[1].to_array(np.float32, (M // 2 + 1, N)), sw.to_array(np.uint16, (M, mlp)), fq.to_array(np.uint16, (M, N)),
                       fm.to_array(np.uint16, (M, mlp))]
    finally:
        L.flux_hip_linear_enable_splitk(1)
        L.flux_hip_linear_force_tile(-1)
        L.flux_hip_linear_probe(-1)
    for a, b in zip(outs[tile], outs[1 if tile == 10 else tile - 8]):
        np.testing.assert_array_equal(a, b)
    lin = oracle_mod.linear(x, W)
    o16, o32, r0, r1, sw, fq, fm = outs[tile]
    assert rel_l2(o32, lin[:, :N]) < 2e-6 and rel_l2(bf16_to_f32(o16), lin[:, :N]) < 4e-3
    assert rel_l2(r0, res[0] + gate * lin[:, :N]) < 2e-6
    assert rel_l2(r1, res[1] + gate * oracle_mod.linear(x2, W[64:64 + N])) < 2e-6
    want_sw = oracle_mod.silu(lin[:, N:N + mlp]) * lin[:, N + mlp:]
    assert rel_l2(bf16_to_f32(sw), want_sw) < 4e-3
    np.testing.assert_array_equal(fq, o16)
    np.testing.assert_array_equal(fm, sw)


def test_linear_rejects_bad_shapes(hip):
    d = hip.DevBuf(1024)
    with pytest.raises(hip.FluxHipError):
        hip.linear(hip.EPI_BF16, [(d.ptr, d.ptr, d.ptr, None, 4)], 128, 100, 100, 100, 128)   # K % 64
    with pytest.raises(hip.FluxHipError):
        hip.linear(hip.EPI_BF16, [(d.ptr, d.ptr, d.ptr, None, 4)], 100, 64, 64, 64, 100)      # N % 128
    with pytest.raises(hip.FluxHipError):
        hip.linear(hip.EPI_RESID, [(d.ptr, d.ptr, d.ptr, None, 4)], 128, 64, 64, 64, 128)     # no gate
    hip.linear(hip.EPI_BF16, [(d.ptr, d.ptr, d.ptr, None, 0)], 128, 64, 64, 64, 128)          # empty is a no-op


@pytest.mark.parametrize("hidden", [256, 3072])
def test_adaln(hip, oracle_mod, hidden):
    rows, split = 45, 17
    x = normal_f32((rows, hidden), 6, 1, 0.5, 3.0)
    m = [normal_f32((hidden,), 6, 2 + i, 0.0, 0.5) for i in range(4)]
    want = np.concatenate([oracle_mod.adaln(x[:split], m[0], m[1]), oracle_mod.adaln(x[split:], m[2], m[3])])
    dx = hip.DevBuf.from_array(x)
    dm = [hip.DevBuf.from_array(v) for v in m]
    out = hip.DevBuf(rows * hidden * 2)
    hip.check(hip.lib().flux_hip_adaln_norm(out.ptr, hidden, dx.ptr, rows, hidden, split,
                                            dm[0].ptr, dm[1].ptr, dm[2].ptr, dm[3].ptr, 1e-6))
    got = bf16_to_f32(out.to_array(np.uint16, (rows, hidden)))
    assert rel_l2(got, want) < 4e-3           # bf16 output rounding
    assert np.abs(got - want).max() < 0.05


@pytest.mark.parametrize("silu", [0, 1])
def test_gemv(hip, oracle_mod, silu):
    M, N, K = 11, 77, 256
    x = normal_f32((M, K), 7, 1, 0.0, 2.0)
    W = q(normal_f32((N, K), 7, 2, 0.0, 0.1))
    want = oracle_mod.linear(oracle_mod.silu(x) if silu else x, W)
    dx, dW = hip.DevBuf.from_array(x), dev_bf16(hip, W)
    out = hip.DevBuf(M * N * 4)
    hip.check(hip.lib().flux_hip_gemv(out.ptr, dx.ptr, dW.ptr, M, N, K, silu))
    assert rel_l2(out.to_array(np.float32, (M, N)), want) < 5e-6


def _attention_case(hip, oracle_mod, n, split, heads, seed, qk_scale=1.0, qkv=None, w=None):
    """qkv buffer -> qk_prepare -> attention, against qk_norm + rope + attention of the oracle."""
    H = heads * 128
    if qkv is None:
        qkv = q(normal_f32((n, 3 * H), seed, 1))
    if w is None:
        w = [normal_f32((128,), seed, 2 + i, 1.0, 0.3) * qk_scale for i in range(4)]   # q0 q1 k0 k1
    ic, isn = oracle_mod.rope_image(1, n - split) if n > split else (np.zeros((0, 128), np.float32),) * 2
    tc, ts = oracle_mod.rope_text(split)
    cos = np.concatenate([tc, ic]) if split else ic
    sin = np.concatenate([ts, isn]) if split else isn
    Q, K, V = qkv[:, :H].copy(), qkv[:, H:2 * H].copy(), qkv[:, 2 * H:].copy()
    for lo, hi, qw, kw in ((0, split, w[0], w[2]), (split, n, w[1], w[3])):
        if hi > lo:
            Q[lo:hi], K[lo:hi] = oracle_mod.qk_norm(Q[lo:hi], K[lo:hi], qw, kw, heads, 128)
    Q = oracle_mod.apply_rope(Q, cos, sin, heads, 128)
    K = oracle_mod.apply_rope(K, cos, sin, heads, 128)
    want = oracle_mod.attention(Q, K, V, heads, 128)

    dqkv = dev_bf16(hip, qkv)
    dw = [hip.DevBuf.from_array(v.astype(np.float32)) for v in w]
    dcos, dsin = hip.DevBuf.from_array(cos), hip.DevBuf.from_array(sin)
    kn = hip.DevBuf(n * H * 2)
    ldo = H + 64
    out = hip.DevBuf.from_array(np.zeros((n, ldo), np.uint16))
    L = hip.lib()
    hip.check(L.flux_hip_qk_prepare(kn.ptr, dqkv.ptr, 3 * H, 0, H, n, heads, split, dw[0].ptr, dw[1].ptr, dw[2].ptr, dw[3].ptr,
                                    dcos.ptr, dsin.ptr, 1e-6))
    hip.check(L.flux_hip_attention(out.ptr, ldo, dqkv.ptr, 3 * H, kn.ptr, dqkv.at(2 * H * 2), 3 * H, n, n, heads))
    # prepared K; prepared Q in place, scaled by 1/sqrt(128) and log2(e); V untouched
    kn_h = bf16_to_f32(kn.to_array(np.uint16, (n, H)))
    assert rel_l2(kn_h, K) < 4e-3
    after = bf16_to_f32(dqkv.to_array(np.uint16, (n, 3 * H)))
    assert rel_l2(after[:, :H], Q * np.float32(0.08838834764831845 * 1.4426950408889634)) < 4e-3
    assert np.array_equal(after[:, H:], qkv[:, H:])
    got = bf16_to_f32(out.to_array(np.uint16, (n, ldo)))
    assert not got[:, H:].any()
    return got[:, :H], want


# (the key loop is written out for four tiles of 64 keys, with up to three more pairs of steps behind it: 300, 440 and 1100 keys
# are 5, 7 and 18 tiles, i.e. three, one and no pairs left over; the others leave none or two)
@pytest.mark.parametrize("n,split,heads", [(1, 0, 1), (64, 64, 2), (80, 64, 2), (191, 50, 3), (300, 100, 2), (333, 128, 2), (440, 128, 2),
                                           (768, 512, 2), (1100, 512, 2)])
def test_attention(hip, oracle_mod, n, split, heads):
    got, want = _attention_case(hip, oracle_mod, n, split, heads, 8)
    # q, k, p are rounded to bf16 inside the kernel and the output is bf16
    assert rel_l2(got, want) < 1e-2, rel_l2(got, want)


def test_attention_sharp_logits(hip, oracle_mod):
    """Norm weights of 3 give logits of order 10: softmax far from uniform, RoPE decisive."""
    got, want = _attention_case(hip, oracle_mod, 200, 72, 2, 9, qk_scale=3.0)
    assert rel_l2(got, want) < 2.5e-2, rel_l2(got, want)


@pytest.mark.parametrize("n,split", [(4608, 512), (2560, 512)])
def test_attention_full_shape_sharp(hip, oracle_mod, n, split):
    """24 heads at the benchmark's sequence lengths (1024x1024: 4096 + 512 tokens; 512x512 with a reference image:
    2048 + 512) with norm weights of 2, i.e. logits of order four: what the whole-model tests with N(0, 0.02)
    norm weights cannot see - RoPE, QK-norm and the online softmax across 72 / 40 key tiles, the 256-query
    workgroups, query blocks of two lengths per head (the automatic mix), heads dealt to the XCDs three at a time."""
    got, want = _attention_case(hip, oracle_mod, n, split, 24, 40, qk_scale=2.0)
    assert rel_l2(got, want) < 2e-2, rel_l2(got, want)
    # per head, so that one wrong head among 24 cannot hide in the total
    for h in range(24):
        r = rel_l2(got[:, h * 128:(h + 1) * 128], want[:, h * 128:(h + 1) * 128])
        assert r < 2.5e-2, (h, r)


@pytest.mark.parametrize("variant", [0, 1])
def test_attention_query_subrange(hip, oracle_mod, variant):
    """seq_q != seq_k: queries are a row range of the sequence (the reference's joint attention asks for the image and
    the text queries separately against all keys, flux_transformer.c:1335-1460). Q and K are prepared once for the whole
    sequence; the q and output pointers move to the range's first row. The rows agree with those of the full call up to bf16
    rounding (which queries share a wave decides when the running maximum is re-based, so not bit for bit)."""
    L = hip.lib()
    L.flux_hip_attention_force_variant(variant)
    try:
        n, split, heads = 700, 200, 3
        H = heads * 128
        qkv = q(normal_f32((n, 3 * H), 44, 1))
        w = [normal_f32((128,), 44, 2 + i, 1.5, 0.3) for i in range(4)]
        ic, isn = oracle_mod.rope_image(20, 25)
        tc, ts = oracle_mod.rope_text(split)
        cos, sin = np.concatenate([tc, ic]), np.concatenate([ts, isn])
        dqkv = dev_bf16(hip, qkv)
        dw = [hip.DevBuf.from_array(v) for v in w]
        dcos, dsin = hip.DevBuf.from_array(cos), hip.DevBuf.from_array(sin)
        kn, dv = hip.DevBuf(n * H * 2), dqkv.at(2 * H * 2)
        hip.check(L.flux_hip_qk_prepare(kn.ptr, dqkv.ptr, 3 * H, 0, H, n, heads, split, dw[0].ptr, dw[1].ptr, dw[2].ptr, dw[3].ptr,
                                        dcos.ptr, dsin.ptr, 1e-6))
        full = hip.DevBuf(n * H * 2)
        hip.check(L.flux_hip_attention(full.ptr, H, dqkv.ptr, 3 * H, kn.ptr, dv, 3 * H, n, n, heads))
        full_h = full.to_array(np.uint16, (n, H))
        Q, K, V = qkv[:, :H].copy(), qkv[:, H:2 * H].copy(), qkv[:, 2 * H:].copy()
        for lo, hi, qw, kw in ((0, split, w[0], w[2]), (split, n, w[1], w[3])):
            Q[lo:hi], K[lo:hi] = oracle_mod.qk_norm(Q[lo:hi], K[lo:hi], qw, kw, heads, 128)
        want = oracle_mod.attention(oracle_mod.apply_rope(Q, cos, sin, heads, 128), oracle_mod.apply_rope(K, cos, sin, heads, 128), V, heads, 128)
        assert rel_l2(bf16_to_f32(full_h), want) < 1.5e-2
        # text queries only, image queries only, a range that starts inside the text and is not a multiple of anything
        for a, b in ((0, split), (split, n), (137, 431), (699, 700)):
            part = hip.DevBuf.from_array(np.full((b - a, H), 0x7fc0, np.uint16))
            hip.check(L.flux_hip_attention(part.ptr, H, dqkv.at(a * 3 * H * 2), 3 * H, kn.ptr, dv, 3 * H, b - a, n, heads))
            got = bf16_to_f32(part.to_array(np.uint16, (b - a, H)))
            assert np.isfinite(got).all()
            assert rel_l2(got, bf16_to_f32(full_h[a:b])) < 4e-3, (a, b)
            assert rel_l2(got, want[a:b]) < 1.5e-2, (a, b)
    finally:
        L.flux_hip_attention_force_variant(-1)


@pytest.mark.parametrize("variant", [-1, 0, 1, 11, 12, 13, 14])
def test_attention_first_key_tile_far_below_the_rest(hip, oracle_mod, variant):
    """Every key of the first tile scores about -1000 (base-2 logits) for every query: the text keys point away from
    all queries and carry a norm weight of 10. The running maximum then starts far below zero; re-basing it must not
    scale the still empty accumulators by 2^1000 (0 * inf). The later keys have logits of order three. The kernels
    with 16 NQ queries per wave fix their references on the first 32 keys and cannot represent the later ones:
    their workgroups notice at the end and compute their queries again with moving references, which must leave the same
    answer."""
    n, split, heads = 192, 64, 1
    u = np.zeros(128, np.float32)
    u[:96] = normal_f32((96,), 46, 1)                 # dims of the RoPE axes that do not turn for text tokens
    qkv = normal_f32((n, 3 * 128), 46, 2)
    qkv[:, :128] = u + 0.05 * qkv[:, :128]            # every query close to u
    qkv[:split, 128:256] = -u + 0.05 * qkv[:split, 128:256]
    w = [np.full(128, 10.0, np.float32), np.full(128, 10.0, np.float32), np.full(128, 10.0, np.float32), np.full(128, 0.3, np.float32)]
    hip.lib().flux_hip_attention_force_variant(variant)
    try:
        got, want = _attention_case(hip, oracle_mod, n, split, heads, 46, qkv=q(qkv), w=w)
        assert np.isfinite(got).all()
        assert rel_l2(got, want) < 2.5e-2, rel_l2(got, want)
        # and an ordinary call right afterwards
        got, want = _attention_case(hip, oracle_mod, 200, 72, 2, 47)
        assert rel_l2(got, want) < 1e-2, rel_l2(got, want)
    finally:
        hip.lib().flux_hip_attention_force_variant(-1)


@pytest.mark.parametrize("lens", [((700, 700), (700, 700)), ((640, 640), (600, 600)), ((300, 300), (2000, 2000)), ((200, 700), (130, 130))])
def test_attention_two_sequences_in_one_launch(hip, lens):
    """flux_hip_attention_batch with two sequences (the two forwards of a CFG step) against one flux_hip_attention call per
    sequence, bit for bit: equal lengths, unequal lengths with the same block plan, lengths whose block plans differ (then
    the batch falls back to a launch per sequence), and a query sub-range in one of them."""
    import ctypes
    L = hip.lib()
    heads = 3
    H = heads * 128
    bufs = []
    for i, (nq, nk) in enumerate(lens):
        qkv = q(normal_f32((nk, 3 * H), 70 + i, 1))
        dqkv = dev_bf16(hip, qkv)
        w = hip.DevBuf.from_array(np.ones(128, np.float32))
        ang = normal_f32((nk, 128), 70 + i, 2)
        dcos, dsin = hip.DevBuf.from_array(np.cos(ang)), hip.DevBuf.from_array(np.sin(ang))
        kn = hip.DevBuf(nk * H * 2)
        hip.check(L.flux_hip_qk_prepare(kn.ptr, dqkv.ptr, 3 * H, 0, H, nk, heads, nk, w.ptr, w.ptr, w.ptr, w.ptr, dcos.ptr, dsin.ptr, 1e-6))
        one = hip.DevBuf.from_array(np.zeros((nq, H), np.uint16))
        hip.check(L.flux_hip_attention(one.ptr, H, dqkv.ptr, 3 * H, kn.ptr, dqkv.at(2 * H * 2), 3 * H, nq, nk, heads))
        both = hip.DevBuf.from_array(np.full((nq, H), 0x7fc0, np.uint16))
        bufs.append((dqkv, kn, one, both, nq, nk, w, dcos, dsin))
    vp2, i2 = ctypes.c_void_p * 2, ctypes.c_int * 2
    out = vp2(*[b[3].ptr for b in bufs])
    qs = vp2(*[b[0].ptr for b in bufs])
    ks = vp2(*[b[1].ptr for b in bufs])
    vs = vp2(*[b[0].at(2 * H * 2) for b in bufs])
    nqs, nks = i2(*[b[4] for b in bufs]), i2(*[b[5] for b in bufs])
    hip.check(L.flux_hip_attention_batch(2, out, H, qs, 3 * H, ks, vs, 3 * H, nqs, nks, heads))
    for dqkv, kn, one, both, nq, nk, *_ in bufs:
        assert np.array_equal(one.to_array(np.uint16, (nq, H)), both.to_array(np.uint16, (nq, H)))


def test_layout_edges_and_updates(hip, oracle_mod):
    C, n = 128, 45
    lat = normal_f32((C, n), 10, 1)
    d = hip.DevBuf.from_array(lat)
    tok = hip.DevBuf(n * C * 2)
    hip.check(hip.lib().flux_hip_latent_to_tokens(tok.ptr, d.ptr, C, n))
    assert np.array_equal(tok.to_array(np.uint16, (n, C)), f32_to_bf16(lat.T.copy()))   # bit exact
    x = normal_f32((1027,), 10, 2)
    dx = hip.DevBuf.from_array(x)
    o = hip.DevBuf(1027 * 2)
    hip.check(hip.lib().flux_hip_f32_to_bf16(o.ptr, dx.ptr, 1027))
    assert np.array_equal(o.to_array(np.uint16, (1027,)), f32_to_bf16(x))               # RNE, bit exact
    z = normal_f32((999,), 10, 3)
    v = normal_f32((999,), 10, 4)
    vu = normal_f32((999,), 10, 5)
    dz, dv, dvu = hip.DevBuf.from_array(z), hip.DevBuf.from_array(v), hip.DevBuf.from_array(vu)
    hip.check(hip.lib().flux_hip_euler_update(dz.ptr, dv.ptr, -0.25, 999))
    np.testing.assert_allclose(dz.to_array(np.float32, (999,)), z + np.float32(-0.25) * v, rtol=0, atol=1e-6)
    dz = hip.DevBuf.from_array(z)
    hip.check(hip.lib().flux_hip_cfg_euler_update(dz.ptr, dvu.ptr, dv.ptr, 4.0, -0.1, 999))
    want = z + np.float32(-0.1) * (vu + np.float32(4.0) * (v - vu))
    np.testing.assert_allclose(dz.to_array(np.float32, (999,)), want, rtol=0, atol=2e-6)


@pytest.mark.parametrize("variant", [-1, 0, 1, 11, 12, 13, 14, 15])
def test_attention_workgroup_variants(hip, oracle_mod, variant):
    """Every kernel variant (32 queries per wave in workgroups of 128 and 256 queries; 16, 32, 48 and 64 queries
    per wave in workgroups of four waves; 15: their automatic mix, as -1) gives the same answer on ragged lengths, from a single key tile up (one, two and three tiles take their own paths
    through the four-slot rings of the wide kernel)."""
    hip.lib().flux_hip_attention_force_variant(variant)
    try:
        for n, split, heads in ((300, 100, 2), (513, 512, 1), (40, 16, 2), (64, 64, 1), (100, 30, 2), (128, 0, 1), (130, 0, 3), (1000, 77, 2)):
            got, want = _attention_case(hip, oracle_mod, n, split, heads, 30 + variant)
            assert rel_l2(got, want) < 1e-2, (n, rel_l2(got, want))
        got, want = _attention_case(hip, oracle_mod, 700, 130, 2, 60 + variant, qk_scale=3.0)     # sharp logits: the maximum moves
        assert rel_l2(got, want) < 2.5e-2, rel_l2(got, want)
    finally:
        hip.lib().flux_hip_attention_force_variant(-1)
