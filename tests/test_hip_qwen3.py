"""GPU parity tests of the Qwen3 text encoder: its two new operators through the C ABI against the CPU
oracle (oracle/qwen3_oracle.c), whole forwards of small encoders against the oracle, and the
full-size encoder against the output of the reference's own qwen3_forward (tests/golden/qwen3_4b.npz).

Tolerances: bf16 operator outputs 4e-3 relative L2 (one rounding); whole forwards rel-L2 <= 2e-2 and
cosine >= 0.999 per captured layer, the gates of the denoising path this output feeds (fp32 residual
stream, bf16 GEMM operands, up to 27 layers).
"""
import os
from dataclasses import replace

import numpy as np
import pytest

from metrics import rel_l2, cosine
from model_spec import (QwenConfig, QWEN3_TINY, QWEN3_4B, make_qwen3_weights, qwen3_tensor_shapes, normal_f32,
                        f32_to_bf16, bf16_to_f32)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    import fluxhip
    fluxhip.init()
    return fluxhip


def q(x):
    return bf16_to_f32(f32_to_bf16(x))


def test_rms_norm(hip, oracle_mod):
    for rows, hidden in ((5, 256), (33, 2560)):
        x = normal_f32((rows, hidden), 71, 1, 0.2, 3.0)
        w = normal_f32((hidden,), 71, 2, 1.0, 0.2)
        dx, dw = hip.DevBuf.from_array(x), hip.DevBuf.from_array(w)
        out = hip.DevBuf(rows * hidden * 2)
        hip.check(hip.lib().flux_hip_rms_norm(out.ptr, dx.ptr, dw.ptr, rows, hidden, 1e-6))
        got = bf16_to_f32(out.to_array(np.uint16, (rows, hidden)))
        assert rel_l2(got, oracle_mod.qwen3_rms_norm(x, w)) < 4e-3


@pytest.mark.parametrize("seq,heads,kv,masked", [(7, 4, 2, 2), (16, 4, 4, 0), (45, 8, 2, 5), (100, 4, 1, 0), (512, 8, 2, 37), (33, 4, 2, -1)])
def test_causal_attention(hip, oracle_mod, seq, heads, kv, masked):
    """masked > 0: that many padding positions at the end; masked = -1: the first position is masked as
    well, so its row has no admissible key and must come out uniform over all columns, as in the reference."""
    qd, kd = heads * 128, kv * 128
    qq = q(normal_f32((seq, qd), 72, 1))
    kk = q(normal_f32((seq, kd), 72, 2))
    vv = q(normal_f32((seq, kd), 72, 3))
    mask = None
    if masked:
        mask = np.ones(seq, np.int32)
        if masked > 0:
            mask[seq - masked:] = 0
        else:
            mask[0] = 0
            mask[seq - 3:] = 0
    want = oracle_mod.qwen3_attention(qq, kk, vv, mask, heads, kv)
    ldv = (seq + 31) // 32 * 32
    qkv = np.concatenate([qq, kk, vv], axis=1)
    vt = np.zeros((kd, ldv), np.float32)
    vt[:, :seq] = vv.T
    dqkv, dvt = hip.DevBuf.from_array(f32_to_bf16(qkv)), hip.DevBuf.from_array(f32_to_bf16(vt))
    dmask = None if mask is None else hip.DevBuf.from_array(mask)
    out = hip.DevBuf(seq * qd * 2)
    hip.check(hip.lib().flux_hip_causal_attention(out.ptr, dqkv.ptr, dvt.ptr, ldv, None if mask is None else dmask.ptr, seq, heads, kv))
    got = bf16_to_f32(out.to_array(np.uint16, (seq, qd)))
    assert rel_l2(got, want) < 6e-3           # probabilities and outputs are each rounded to bf16 once
    if masked == -1:
        assert rel_l2(got[0, :128], vv[:, :128].mean(axis=0)) < 6e-3     # uniform over ALL columns


MID = QwenConfig(hidden=512, intermediate=1152, heads=8, kv_heads=2, layers=6, vocab=1000, out_layers=(0, 3, 5))


@pytest.mark.parametrize("cfg,seq,npad", [(QWEN3_TINY, 7, 2), (QWEN3_TINY, 64, 0), (MID, 100, 13), (MID, 512, 200)])
def test_forward_against_oracle(hip, oracle_mod, cfg, seq, npad):
    W = make_qwen3_weights(cfg)
    dev = hip.Qwen3(cfg, W)
    cpu = oracle_mod.Qwen3Oracle(cfg, W)
    rng = np.random.default_rng(seq)
    ids = rng.integers(0, cfg.vocab, seq).astype(np.int32)
    mask = None
    if npad:
        mask = np.ones(seq, np.int32)
        mask[seq - npad:] = 0
    got = dev.forward(ids, mask)
    want = cpu.forward(ids, mask)
    real = seq - npad
    for j in range(3):
        a, b = got[:real, j * cfg.hidden:(j + 1) * cfg.hidden], want[:real, j * cfg.hidden:(j + 1) * cfg.hidden]
        r, c = rel_l2(a, b), cosine(a, b)
        print(f"qwen3 {cfg.hidden}x{cfg.layers} seq {seq}: layer {cfg.out_layers[j]} rel_l2={r:.3e} cos={c:.6f}", flush=True)
        assert r <= 2e-2 and c >= 0.999
    assert rel_l2(got, want) <= 2e-2          # padded positions included
    # the same call again gives the same bits
    np.testing.assert_array_equal(dev.forward(ids, mask), got)
    dev.close()
    cpu.close()


def test_full_size_against_reference_output(hip, golden_dir):
    """The reference's sizes (27 of the 36 layers are needed) on the synthetic encoder of
    model_spec.make_qwen3_weights; expected values were produced by the reference's qwen3_forward."""
    gold = np.load(os.path.join(golden_dir, "qwen3_4b.npz"))
    cases = {"masked8": ([151644, 872, 198, 64, 8251, 151645, 151643, 151643], [1, 1, 1, 1, 1, 1, 0, 0]),
             "plain5": ([11, 4999, 151935, 0, 77777], None)}
    cfg = QWEN3_4B
    dev = hip.Qwen3(cfg)
    for name in qwen3_tensor_shapes(cfg):
        if name.startswith("model.layers.") and int(name.split(".")[2]) > max(cfg.out_layers):
            continue
        dev.set_tensor(name, make_qwen3_weights(cfg, only=[name])[name])
    for key, (ids, mask) in cases.items():
        got = dev.forward(ids, mask)
        r, c = rel_l2(got, gold[key]), cosine(got, gold[key])
        print(f"qwen3 4B {key}: rel_l2={r:.3e} cos={c:.6f}", flush=True)
        assert r <= 2e-2 and c >= 0.999
    dev.close()


def test_errors(hip):
    L = hip.lib()
    cfg = QWEN3_TINY
    m = hip.Qwen3(cfg, {})
    ids = np.zeros(4, np.int32)
    assert not L.flux_hip_qwen3_forward(m.h, ids.ctypes.data, None, 4)              # nothing loaded
    assert b"embed_tokens" in L.flux_hip_last_error()
    bad = np.zeros(5, np.uint16)
    assert L.flux_hip_qwen3_set_tensor(m.h, b"model.layers.0.input_layernorm.weight", 2, bad.ctypes.data, 5) == 0
    assert L.flux_hip_qwen3_set_tensor(m.h, b"model.layers.0.nonsense", 2, bad.ctypes.data, 5) == 0
    m.close()
    W = make_qwen3_weights(cfg)
    m = hip.Qwen3(cfg, W)
    assert not L.flux_hip_qwen3_forward(m.h, np.zeros(600, np.int32).ctypes.data, None, 600)   # longer than 512
    m.close()
    import ctypes
    c = hip._QwenCfg(256, 384, 4, 2, 64, 5, 300, (ctypes.c_int * 3)(1, 2, 4), 1e6, 1e-6)
    assert not L.flux_hip_qwen3_new(ctypes.byref(c))                                # head_dim 64 is not built
    assert b"head_dim" in L.flux_hip_last_error()
