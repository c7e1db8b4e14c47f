"""Address arithmetic of the operand loaders, replayed on the CPU.

One launch per layer reads activations and weights through plain global loads: no buffer descriptor checks the
offsets there, only the 256 bytes of slack behind every allocation cover what an edge tile reads past a row.  This
file restates, per loader of aspen_amd/csrc/hip/tile_kernels.h, the float offset every lane issues for every K slice
its K loop asks for (including the repeated request for the last slice that the two-deep loops make, which the
stepping convolution loader answers one step past the K axis), on the tile grids the C library really builds for the
micro networks and for a ragged 272-token sequence, and asserts that every offset that is actually requested lies
inside [0, columns * ld + slack).  It also records what the loader of the transposed V operand would request without
its `position < sequence length` guard: rows past the last batch item's sequence, kilobytes beyond the matrix.
"""
import numpy as np
import pytest

from aspen_amd import api, models as M
from tests import helpers as H

SLACK = 64                      # floats every device allocation carries behind its end (aspen_hip_alloc)
BK = 32


def round_up(a, b):
    return (a + b - 1) // b * b


def contraction_geometry(L, info, parent_info):
    """Kp, taps, per-tap channel run and operand kind as dnn.c:aspen_layer_to_device / nasm.c derive them."""
    t = L["type"]
    if t == "conv":
        taps, ic, kw_count = L["size"] * L["size"], L["inC"], L["size"]
    elif t == "fc":
        taps, ic, kw_count = L["inH"] * L["inW"], L["inC"], L["inW"]
    else:
        taps, ic, kw_count = 1, L["K"], 1
    dense3 = t == "conv" and ic == 3 and taps * 3 <= 508 and info["H"] <= 64
    icp = 3 if dense3 else round_up(ic, 4)
    kp = round_up(taps * icp, BK)
    ld0 = parent_info["stride"]
    pointwise = t == "matmul" or (t == "conv" and L["size"] == 1 and L["stride"] == 1 and L["pad"] == 0) or (t == "fc" and taps == 1)
    direct = pointwise and ic % BK == 0 and ld0 >= kp
    return dict(taps=taps, ic=ic, icp=icp, kp=kp, kw_count=kw_count, dense3=dense3, direct=direct, ld0=ld0)


def slices_asked(kbase, kiters, depth):
    """Slice indices a K loop hands to load (): gemm_core / gemm_core_single_block.  With two register sets the
    requests are unconditional and clamped to the last slice (asked for again, answer dropped)."""
    asked = [kbase]
    if depth == 2 and kiters > 1:
        asked.append(kbase + 1)
    if kiters > depth:
        asked.append(kbase + depth)
    for it in range(kiters - 1):
        if depth == 2:
            asked.append(kbase + min(it + 1 + depth, kiters - 1))
        elif it + 1 + depth < kiters:
            asked.append(kbase + it + 1 + depth)
    return asked


def conv_rows(L, n_rows, N, first_row):
    """(base, ih0, iw0) of ConvLoader / Dense3Loader for tile rows first_row .. first_row + n_rows (clamped to N - 1)."""
    OH, OW = (1, 1) if L["type"] == "fc" else (L["H"], L["W"])
    IH, IW = L["inH"], L["inW"]
    stride, pad = (1, 0) if L["type"] == "fc" else (L["stride"], L["pad"])
    n = np.minimum(first_row + np.arange(n_rows), N - 1)
    b, rem = n // (OH * OW), n % (OH * OW)
    oh, ow = rem // OW, rem % OW
    ih0, iw0 = oh * stride - pad, ow * stride - pad
    return b, ih0, iw0, IH, IW


def check(offsets, ok, size, what):
    offsets, ok = np.asarray(offsets, dtype=np.int64), np.asarray(ok, dtype=bool)
    issued = offsets[ok]
    if issued.size:
        assert issued.min() >= 0, f"{what}: offset {issued.min()} below the matrix"
        assert issued.max() + 4 <= size + SLACK, f"{what}: offset {issued.max()} + 4 floats beyond {size} + {SLACK}"
    return int(issued.size)


def walk_contraction(L, info, pinfo, batch, name, l):
    g = contraction_geometry(L, info, pinfo)
    M_, N = info["H"], info["W"]
    bm, bn = info["tile_H"], info["tile_W"]
    tiles_m, tiles_n = info["tiles_H"], (N + bn - 1) // bn
    splits, kiters_all = info["splits"], g["kp"] // BK
    narrow = info["variant"] == 3
    in_cols = N * L["inH"] * L["inW"] if L["type"] == "fc" else (N // (L["H"] * L["W"])) * L["inH"] * L["inW"] if L["type"] == "conv" else N
    in_size = in_cols * g["ld0"]
    w_size = round_up(M_, 128) * g["kp"]
    chunk = np.arange(8)
    count = 0
    for s in range(splits):
        kbase = s * info["kiters_per_split"] if splits > 1 else 0
        kiters = min(info["kiters_per_split"], kiters_all - kbase) if splits > 1 else kiters_all
        assert kiters > 0, (name, l, "empty split")
        for tn in range(tiles_n):
            n0 = tn * bn
            if narrow:
                # narrow_mainloop: wave w takes a contiguous quarter; a lane = (row, K half); requests are exact (guarded by cnt)
                per = (kiters + 3) // 4
                rows = np.arange(32)
                n = np.minimum(n0 + rows, N - 1)
                for w in range(4):
                    w0 = min(w * per, kiters)
                    cnt = min(per, kiters - w0)
                    first = kbase + w0
                    for i in range(cnt):
                        for sub in range(4):
                            for khalf in (0, 4):
                                k = (first + i) * BK + sub * 8 + khalf
                                for tm in range(tiles_m):
                                    a = (tm * 32 + rows) * g["kp"] + k
                                    count += check(a, np.ones(32, bool), w_size, f"{name} layer {l} narrow weights")
                                if g["direct"]:
                                    count += check(n * g["ld0"] + k, np.ones(32, bool), in_size, f"{name} layer {l} narrow direct")
                                else:
                                    block, tap = (first + i) // g["taps"], (first + i) % g["taps"]
                                    c = block * BK
                                    kh, kw = tap // g["kw_count"], tap % g["kw_count"]
                                    b, ih0, iw0, IH, IW = conv_rows(L, 32, N, n0)
                                    base = ((b * IH + ih0) * IW + iw0) * g["ld0"]
                                    ok = (ih0 + kh >= 0) & (ih0 + kh < IH) & (iw0 + kw >= 0) & (iw0 + kw < IW)
                                    count += check(base + (kh * IW + kw) * g["ld0"] + c + sub * 8 + khalf, ok, in_size, f"{name} layer {l} narrow taps")
                continue
            depth = 2 if (L["type"] == "matmul" and bm == 64 and bn == 64) or info["variant"] == 4 else 1      # (VAR2_DEPTH of the transformer kernels, VAR4_DEPTH)
            asked = slices_asked(kbase, kiters, depth)
            rows_b = np.arange(bn)
            # weights: RowLoader<BM>, rows padded to a multiple of 128
            for tm in range(tiles_m):
                for it in asked:
                    a = ((tm * bm + np.arange(bm))[:, None] * g["kp"] + chunk[None, :] * 4 + it * BK).ravel()
                    count += check(a, np.ones(a.size, bool), w_size, f"{name} layer {l} weights")
            if g["direct"]:
                # ActRowLoader: rows clamped to N - 1
                r = np.minimum(n0 + rows_b, N - 1)
                for it in asked:
                    o = (r[:, None] * g["ld0"] + chunk[None, :] * 4 + it * BK).ravel()
                    count += check(o, np.ones(o.size, bool), in_size, f"{name} layer {l} direct operand")
                continue
            b, ih0, iw0, IH, IW = conv_rows(L, bn, N, n0)
            base = ((b * IH + ih0) * IW + iw0) * g["ld0"]
            if g["dense3"]:
                # Dense3Loader: chunk kc spans taps 4kc // 3 and the next; two 16-byte loads per chunk
                for it in asked:
                    for ch in range(8):
                        kc = it * 8 + ch
                        for e in range(2):
                            tap = (kc * 4) // 3 + e
                            if tap >= g["taps"]:
                                kh, kw, off = 0x4000, 0, 0
                            else:
                                kh, kw = tap // g["kw_count"], tap % g["kw_count"]
                                off = (kh * IW + kw) * g["ld0"]
                            ok = (ih0 + kh >= 0) & (ih0 + kh < IH) & (iw0 + kw >= 0) & (iw0 + kw < IW)
                            count += check(base + off, ok, in_size, f"{name} layer {l} dense3")
            elif g["ic"] % BK != 0:
                # ConvLoader<TABLE>: k-chunk table, chunks beyond the real K carry kh = 0x4000 (never in range)
                for it in asked:
                    for ch in range(8):
                        c = it * 8 + ch
                        tap, chan = (c * 4) // g["icp"], (c * 4) % g["icp"]
                        if tap >= g["taps"]:
                            kh, kw, off = 0x4000, 0, 0
                        else:
                            kh, kw = tap // g["kw_count"], tap % g["kw_count"]
                            off = (kh * IW + kw) * g["ld0"] + chan
                        ok = (ih0 + kh >= 0) & (ih0 + kh < IH) & (iw0 + kw >= 0) & (iw0 + kw < IW)
                        count += check(base + off, ok, in_size, f"{name} layer {l} table")
            else:
                # ConvLoader stepping: the position advances by one slice per request, whatever `it` says; the
                # repeated requests of a two-deep loop therefore land one and two steps past the K axis.  K order:
                # (channel block of 32, kh, kw, channel in block), so a step past the end is the first taps again at
                # the 32 channels BEHIND the pixel's run
                pos = kbase
                for _ in asked:
                    block, tap = pos // g["taps"], pos % g["taps"]
                    c = block * BK
                    kh, kw = tap // g["kw_count"], tap % g["kw_count"]
                    ok = (ih0 + kh >= 0) & (ih0 + kh < IH) & (iw0 + kw >= 0) & (iw0 + kw < IW)
                    o = (base + (kh * IW + kw) * g["ld0"] + c)[:, None] + chunk[None, :] * 4
                    count += check(o.ravel(), np.repeat(ok, 8), in_size, f"{name} layer {l} stepping tap {tap}")
                    pos += 1
    return count


def walk_attention(L, info, infos, batch, seq, name, l, unguarded=False):
    """K tile: ActRowLoader over Key and Query rows (clamped to the sequence's last row).  V tile: TransLoader64 over the
    Value matrix (rows = positions, guarded by position < seq) and ActRowLoader over the probabilities."""
    S, H_ = seq, L["n_head"]
    hd = L["n_embd"] // H_
    count, worst = 0, 0
    chunk = np.arange(8)
    if L["type"] == "attn_k":
        q, k = infos[L["p0"]], infos[L["p1"]]
        for b in range(batch):
            for h in range(H_):
                for q0 in range(0, S, info["tile_W"]):
                    for k0 in range(0, S, 128):
                        for rows, first, pinfo in ((128, b * S + k0, k), (info["tile_W"], b * S + q0, q)):
                            r = np.minimum(first + np.arange(rows), b * S + S - 1)
                            for it in range(hd // BK):
                                o = (r[:, None] * pinfo["stride"] + h * hd + chunk[None, :] * 4 + it * BK).ravel()
                                count += check(o, np.ones(o.size, bool), pinfo["W"] * pinfo["stride"], f"{name} layer {l} K-attention")
        return count, worst
    p, v = infos[L["p0"]], infos[L["p1"]]
    ld1, tile_m = v["stride"], info["tile_H"]
    c4, s0 = np.arange(256) & 15, np.arange(256) >> 4
    v_size = v["W"] * v["stride"]
    for b in range(batch):
        for m0 in range(0, info["H"], tile_m):
            h = m0 // hd
            prow = (b * H_ + h) * S
            first = b * S * ld1 + m0
            live = c4 * 4 < tile_m
            for it in range((S + BK - 1) // BK):
                for half in (0, 16):
                    s = it * BK + s0 + half
                    o = first + (s0 + half) * ld1 + c4 * 4 + it * BK * ld1
                    ok = live & (s < S)
                    if unguarded:
                        worst = max(worst, int((o[live] + 4).max()) - v_size)
                    else:
                        count += check(o, ok, v_size, f"{name} layer {l} V operand")
            for q0 in range(0, S, info["tile_W"]):
                r = np.minimum(prow + q0 + np.arange(info["tile_W"]), prow + S - 1)
                for it in range((S + BK - 1) // BK):
                    o = (r[:, None] * p["stride"] + chunk[None, :] * 4 + it * BK).ravel()
                    count += check(o, np.ones(o.size, bool), p["W"] * p["stride"], f"{name} layer {l} probabilities")
    return count, worst


def walk_network(name, cfg, batch, seq, min_ninst):
    layers = M.parse_cfg(cfg)
    d = api.Dnn(cfg, None)
    n = api.Nasm(d, batch, seq, min_ninst)
    infos = [n.info(l) for l in range(n.num_ldata)]
    total = 0
    try:
        for l, L in enumerate(layers):
            if infos[l]["num_ninst"] == 0:
                continue
            if L["type"] in ("conv", "fc", "matmul"):
                total += walk_contraction(L, infos[l], infos[L["p0"]], batch, name, l)
            elif L["type"] in ("attn_k", "attn_v"):
                total += walk_attention(L, infos[l], infos, batch, seq, name, l)[0]
    finally:
        n.destroy(); d.destroy()
    return total


@pytest.mark.parametrize("min_ninst", [8, 32, 1024])
@pytest.mark.parametrize("name", list(H.micro_cases()))
def test_every_requested_operand_offset_lies_inside_its_matrix(name, min_ninst):
    cfg, style, batch, seq, seed, kind = H.micro_cases()[name]
    assert walk_network(name, cfg, batch, seq, min_ninst) > 0


@pytest.mark.parametrize("min_ninst", [1, 8])
@pytest.mark.parametrize("name", ["vgg_mini_b5", "custom_b3", "resnet_mini_b2"])
def test_tall_tiles_stay_inside_their_matrices(name, min_ninst, monkeypatch):
    """The same walk with the 128 x 32 shape on every layer of at most 32 columns (the size limit lowered)."""
    monkeypatch.setenv("ASPEN_GPU_WEIGHT_STREAM_BYTES", "0")
    cfg, style, batch, seq, seed, kind = H.micro_cases()[name]
    assert walk_network(name, cfg, batch, seq, min_ninst) > 0


@pytest.mark.parametrize("masked", [0, 1])
def test_ragged_272_token_sequence_stays_inside_its_matrices(masked):
    cfg = M.gpt2_cfg(1, 128, 2, 256) if masked else M.bert_cfg(1, 128, 2, 256)
    assert walk_network("ragged", cfg, 1, 272, 64) > 0


def test_transposed_v_operand_needs_its_sequence_guard():
    """What the V loader would request if positions >= the sequence length were not masked out before the load (the
    variant that replaced the branch by an out-of-range offset, which only a buffer descriptor turns into zeros): for
    24 tokens the last K slice covers positions 24 .. 31, i.e. for the last batch item 8 rows of ld floats behind the
    matrix -- 4 KB with a stride of 128, far beyond the 256 bytes of slack, so plain global loads (one launch per
    layer) would read whatever follows the Value matrix in the arena, or fault where nothing does."""
    cfg, style, batch, seq, seed, kind = H.micro_cases()["bert_mini_b2_s24"]
    layers = M.parse_cfg(cfg)
    d = api.Dnn(cfg, None)
    n = api.Nasm(d, batch, seq, 32)
    infos = [n.info(l) for l in range(n.num_ldata)]
    try:
        l = next(i for i, L in enumerate(layers) if L["type"] == "attn_v")
        _, worst = walk_attention(layers[l], infos[l], infos, batch, seq, "bert_mini", l, unguarded=True)
        v = infos[layers[l]["p1"]]
        rows_past = round_up(seq, BK) - seq
        assert worst == rows_past * v["stride"] - (v["stride"] - layers[l]["C"]), (worst, rows_past, v["stride"])
        assert worst * 4 > 256                                     # bytes beyond the matrix: more than the slack
        guarded, _ = walk_attention(layers[l], infos[l], infos, batch, seq, "bert_mini", l)
        assert guarded > 0                                         # with the guard every request is inside
    finally:
        n.destroy(); d.destroy()
