"""Pins the CPU oracle (oracle/aspen_oracle.c) against mathematics it did not come from:
library routines (torch.nn.functional on CPU), brute force on tiny inputs, closed forms and
invariants.  A dropped term, wrong sign / index or transposed operand fails at least one of them."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import cpu

RNG = np.random.default_rng(1234)


def rnd(*shape, scale=1.0):
    return (RNG.standard_normal(shape) * scale).astype(np.float32)


# ---- packed weights + micro-kernel --------------------------------------------------------------
@pytest.mark.parametrize("M,K", [(8, 5), (13, 7), (1, 1), (24, 368), (129, 33)])
def test_pack_weight_index_identity(M, K):
    w = rnd(M, K)
    p = cpu.pack_weight(w)
    assert p.size == ((M + 7) // 8) * K * 8
    for m in (0, M // 2, M - 1):
        for k in (0, K // 2, K - 1):
            assert p[((m // 8) * K + k) * 8 + m % 8] == w[m, k]
    # padding rows of the last group are zero
    if M % 8:
        last = p.reshape(-1, K, 8)[-1]
        assert np.all(last[:, M % 8:] == 0)


@pytest.mark.parametrize("M,N,K", [(8, 12, 8), (13, 11, 37), (1, 1, 1), (130, 7, 369), (64, 25, 100)])
def test_sgemm_packed_brute_force(M, N, K):
    """C[n][m] += sum_k A[m][k] B[n][k], remainders in M (not /8), N (not /4) and K."""
    A, B = rnd(M, K), rnd(N, K)
    C0 = rnd(N, M)
    got = cpu.sgemm_packed(cpu.pack_weight(A), B, M, C0)
    want = C0.astype(np.float64) + B.astype(np.float64) @ A.astype(np.float64).T
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)
    # transposed operand would give a different (or ill-shaped) result
    if M != N:
        assert got.shape == (N, M)


# ---- activations ---------------------------------------------------------------------------------
def test_activations_closed_forms():
    x = np.array([-3.0, -1.0, -0.1, 0.0, 0.1, 1.0, 3.0], dtype=np.float32)
    t = torch.from_numpy(x)
    assert np.array_equal(cpu.activate(x, 0), x) and np.array_equal(cpu.activate(x, 2), x)
    assert np.array_equal(cpu.activate(x, 4), np.maximum(x, 0))
    assert np.allclose(cpu.activate(x, 5), np.where(x > 0, x, 0.1 * x), rtol=1e-6)
    assert np.allclose(cpu.activate(x, 6), np.where(x > 0, x, 0.1 * (np.exp(x.astype(np.float64)) - 1)), rtol=1e-6)
    assert np.allclose(cpu.activate(x, 7), np.where(x > 0, 1.0507 * x, 1.0507 * 1.67326 * (np.exp(x.astype(np.float64)) - 1)), rtol=1e-6)
    # the same two against the library forms: ELU with the reference's alpha 0.1; SELU, whose published
    # constants (1.0507009873554805, 1.6732632423543772) the reference rounds to 1.0507 and 1.67326
    assert np.allclose(cpu.activate(x, 6), F.elu(t, alpha=0.1).numpy(), rtol=1e-6, atol=1e-7)
    assert np.allclose(cpu.activate(x, 7), F.selu(t).numpy(), rtol=3e-6, atol=1e-7)
    assert not np.allclose(cpu.activate(x, 6), F.elu(t, alpha=1.0).numpy(), rtol=1e-3)       # alpha is discriminated
    assert np.allclose(cpu.activate(x, 1), torch.sigmoid(t).numpy(), rtol=1e-6)
    assert np.allclose(cpu.activate(x, 3), torch.tanh(t).numpy(), rtol=1e-6)
    assert np.allclose(cpu.activate(x, 8), F.gelu(t).numpy(), rtol=1e-5, atol=2e-6)      # float erff
    assert np.allclose(cpu.activate(x, 9), F.gelu(t, approximate="tanh").numpy(), rtol=1e-5, atol=2e-6)


# ---- conv / pools against torch ------------------------------------------------------------------
def nhwc(x_nchw):
    b, c, h, w = x_nchw.shape
    return np.ascontiguousarray(x_nchw.transpose(0, 2, 3, 1)).reshape(b * h * w, c)


def to_nchw(cols, b, h, w):
    return cols.reshape(b, h, w, -1).transpose(0, 3, 1, 2)


@pytest.mark.parametrize("B,C,H,W,OC,k,s,p,act", [
    (2, 3, 9, 11, 5, 3, 1, 1, 4), (1, 8, 7, 7, 16, 1, 1, 0, 0), (2, 4, 10, 10, 6, 3, 2, 1, 4),
    (1, 3, 12, 12, 7, 7, 2, 3, 4), (3, 5, 6, 5, 9, 5, 1, 2, 0), (1, 16, 8, 8, 8, 1, 2, 0, 0)])
def test_conv2d_matches_torch(B, C, H, W, OC, k, s, p, act):
    x, w, b = rnd(B, C, H, W), rnd(OC, C, k, k, scale=0.3), rnd(OC, scale=0.1)
    got = cpu.conv2d(nhwc(x), w, b, B, H, W, s, p, act)
    want = F.conv2d(torch.from_numpy(x), torch.from_numpy(w), torch.from_numpy(b), stride=s, padding=p)
    if act == 4:
        want = F.relu(want)
    OH, OW = want.shape[2], want.shape[3]
    assert np.allclose(to_nchw(got, B, OH, OW), want.numpy(), rtol=1e-4, atol=1e-5)


def test_conv_special_cases():
    # zero input -> act(bias); 1x1 conv == matmul over channels
    B, C, H, W, OC = 1, 4, 5, 5, 6
    w, b = rnd(OC, C, 3, 3), rnd(OC)
    z = cpu.conv2d(np.zeros((B * H * W, C), np.float32), w, b, B, H, W, 1, 1, 4)
    assert np.allclose(z, np.maximum(b, 0)[None, :].repeat(B * H * W, 0))
    x, w1 = rnd(B * H * W, C), rnd(OC, C, 1, 1)
    assert np.allclose(cpu.conv2d(x, w1, b, B, H, W, 1, 0, 0), cpu.matmul(x, w1.reshape(OC, C), b, 0), rtol=1e-6)


@pytest.mark.parametrize("k,s,p", [(2, 2, 0), (3, 2, 1), (3, 1, 1)])
def test_pools_match_torch(k, s, p):
    B, C, H, W = 2, 6, 9, 8
    x = rnd(B, C, H, W)
    t = torch.from_numpy(x)
    mp = cpu.pool("maxpool", nhwc(x), B, H, W, C, k, s, p, 0)
    ap = cpu.pool("avgpool", nhwc(x), B, H, W, C, k, s, p, 0)
    wm = F.max_pool2d(t, k, s, p)
    wa = F.avg_pool2d(t, k, s, p, count_include_pad=True)     # padded taps count in the divisor
    assert np.array_equal(to_nchw(mp, B, wm.shape[2], wm.shape[3]), wm.numpy())
    assert np.allclose(to_nchw(ap, B, wa.shape[2], wa.shape[3]), wa.numpy(), rtol=1e-6, atol=1e-7)
    # all-negative input: max-pool padding must not contribute zeros
    neg = -np.abs(x) - 1
    mpn = cpu.pool("maxpool", nhwc(neg), B, H, W, C, k, s, p, 0)
    assert mpn.max() < 0


def test_fc_is_matmul_over_hwc_flatten():
    B, C, H, W, OC = 3, 5, 4, 3, 7
    x, w, b = rnd(B, C, H, W), rnd(OC, C, H, W), rnd(OC)
    got = cpu.fc(nhwc(x), w, b, B, 4)
    want = F.relu(F.linear(torch.from_numpy(x).reshape(B, -1), torch.from_numpy(w).reshape(OC, -1), torch.from_numpy(b)))
    assert np.allclose(got, want.numpy(), rtol=1e-4, atol=1e-5)


# ---- elementwise / normalisation ----------------------------------------------------------------
def test_residual_layernorm_softmax():
    N, M = 11, 24
    a, b = rnd(N, M), rnd(N, M)
    assert np.array_equal(cpu.residual(a, b, 4), np.maximum(a + b, 0))
    g, beta = rnd(M), rnd(M)
    ln = cpu.layernorm(a, g, beta)
    want = F.layer_norm(torch.from_numpy(a), (M,), torch.from_numpy(g), torch.from_numpy(beta), eps=1e-6)
    assert np.allclose(ln, want.numpy(), rtol=1e-4, atol=1e-5)
    # small-variance input separates eps = 1e-6 from 1e-12 and from 1e-5
    tiny = (a * 1e-3).astype(np.float32)
    for eps, ok in ((1e-6, True), (1e-12, False), (1e-5, False)):
        w2 = F.layer_norm(torch.from_numpy(tiny), (M,), torch.from_numpy(g), torch.from_numpy(beta), eps=eps).numpy()
        assert np.allclose(cpu.layernorm(tiny, g, beta), w2, rtol=1e-3, atol=1e-4) == ok
    sm = cpu.softmax(a)
    assert np.allclose(sm, F.softmax(torch.from_numpy(a), dim=1).numpy(), rtol=1e-5, atol=1e-7)
    assert np.allclose(sm.sum(1), 1, atol=1e-5)


# ---- attention -----------------------------------------------------------------------------------
@pytest.mark.parametrize("masked", [0, 1])
def test_attention_matches_textbook(masked):
    B, H, S, hd = 2, 3, 10, 8
    E = H * hd
    q, k, v = rnd(B * S, E, scale=0.5), rnd(B * S, E, scale=0.5), rnd(B * S, E)
    p = cpu.k_attention(q, k, B, H, S, masked)              # [B*H*S queries][S keys]
    qt = torch.from_numpy(q).reshape(B, S, H, hd).permute(0, 2, 1, 3)
    kt = torch.from_numpy(k).reshape(B, S, H, hd).permute(0, 2, 1, 3)
    vt = torch.from_numpy(v).reshape(B, S, H, hd).permute(0, 2, 1, 3)
    scores = qt @ kt.transpose(-1, -2) / math.sqrt(hd)
    if masked:
        scores = scores.masked_fill(torch.triu(torch.ones(S, S, dtype=torch.bool), 1), float("-inf"))
    want_p = torch.softmax(scores, -1)                       # [B][H][q][key]
    assert np.allclose(p.reshape(B, H, S, S), want_p.numpy(), rtol=1e-4, atol=1e-6)
    assert np.allclose(p.sum(1), 1, atol=1e-5)
    if masked:
        pm = p.reshape(B, H, S, S)
        assert np.all(pm[:, :, np.triu_indices(S, 1)[0], np.triu_indices(S, 1)[1]] == 0)   # exactly zero
        assert np.allclose(pm[:, :, 0, 0], 1)                                              # first row one-hot
    o = cpu.v_attention(p, v, B, H, S)
    want_o = (want_p @ vt).permute(0, 2, 1, 3).reshape(B * S, E)
    assert np.allclose(o, want_o.numpy(), rtol=1e-4, atol=1e-6)


# ---- detection layers ------------------------------------------------------------------------------
def test_yolo_and_append_match_torch():
    B, IH, IW, R, A, stride = 2, 3, 4, 7, 3, 8
    x = rnd(B, A * R, IH, IW)
    anchors = np.array([10, 13, 16, 30, 33, 23], dtype=np.float32)
    got = cpu.yolo(nhwc(x), anchors, B, IH, IW, R, stride)           # [(b, a, h, w)][R]
    t = torch.from_numpy(x).reshape(B, A, R, IH, IW)
    gx = torch.arange(IW).float().view(1, 1, 1, IW)
    gy = torch.arange(IH).float().view(1, 1, IH, 1)
    want = torch.empty_like(t)
    want[:, :, 0] = (torch.sigmoid(t[:, :, 0]) + gx) * stride
    want[:, :, 1] = (torch.sigmoid(t[:, :, 1]) + gy) * stride
    want[:, :, 2] = torch.exp(t[:, :, 2]) * torch.tensor(anchors[0::2]).view(1, A, 1, 1)
    want[:, :, 3] = torch.exp(t[:, :, 3]) * torch.tensor(anchors[1::2]).view(1, A, 1, 1)
    want[:, :, 4:] = torch.sigmoid(t[:, :, 4:])
    want = want.permute(0, 1, 3, 4, 2).reshape(B * A * IH * IW, R)
    assert np.allclose(got, want.numpy(), rtol=1e-5, atol=1e-6)
    # append = nearest upsampling of the first operand, channel concatenation with the second
    a, b = rnd(B, 5, 3, 2), rnd(B, 4, 6, 4)
    got = cpu.append(nhwc(a), nhwc(b), B, 6, 4, 2)
    want = torch.cat([F.interpolate(torch.from_numpy(a), scale_factor=2, mode="nearest"), torch.from_numpy(b)], dim=1)
    assert np.array_equal(to_nchw(got, B, 6, 4), want.numpy())
