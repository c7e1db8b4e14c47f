"""Host-side logic of the C library, no GPU needed: cfg parsing, out_mat geometry, the tile grid and
the tile dependency graph (checked against a brute-force derivation from the layer semantics), FLOP
accounting (against the totals in the reference's shipped .nasm headers) and error behaviour."""
import os

import numpy as np
import pytest

from aspen_amd import api, models as M
from tests import helpers as H

# TOTAL_FLOPS of the reference's shipped graphs (files/resnet50/resnet50_B1.nasm:5, files/vgg16/vgg16_B1.nasm:5)
REF_TOTAL_FLOPS = {"resnet50": 8185945088, "vgg16": 30946800640}


def make(case, min_ninst):
    cfg, layers, tens, x, batch, seq = H.build_case(case)
    d = api.Dnn(cfg, None)
    return layers, d, api.Nasm(d, batch, seq, min_ninst), batch, seq


def test_total_flops_match_reference_headers():
    for gen, key in ((M.resnet50_cfg, "resnet50"), (M.vgg16_cfg, "vgg16")):
        d = api.Dnn(gen(), None)
        n = api.Nasm(d, 1, 0, 64)
        assert n.total_flops == REF_TOTAL_FLOPS[key]
        n.destroy(); d.destroy()
    # 64-bit accounting: batch 32 is exactly 32x batch 1 (the reference's 32-bit sum overflows here)
    d = api.Dnn(M.resnet50_cfg(), None)
    n = api.Nasm(d, 32, 0, 64)
    assert n.total_flops == 32 * REF_TOTAL_FLOPS["resnet50"] == 261950242816
    n.destroy(); d.destroy()


def test_out_mat_geometry_matches_cfg():
    """rows = channels (or S for K-attention), columns = batch x positions; stride >= rows, multiple of 4."""
    for name, case in H.micro_cases().items():
        layers, d, n, batch, seq = make(case, 64)
        assert n.num_ldata == len(layers)
        for l, L in enumerate(layers):
            i = n.info(l)
            assert api.LAYER_TYPE_NAMES[i["type"]] == L["type"], (name, l)
            if L["type"] == "attn_k":
                assert (i["H"], i["W"]) == (seq, batch * L["n_head"] * seq)
            elif seq:
                assert (i["H"], i["W"]) == (L["C"], batch * seq)
            else:
                assert (i["H"], i["W"]) == (L["C"], batch * L["H"] * L["W"])
            assert i["stride"] >= i["H"] and i["stride"] % 4 == 0
        n.destroy(); d.destroy()


def needed_regions(L, layers, c0, c1, r0, r1, batch, seq):
    """Brute force from the layer semantics: for output columns [c0,c1) x rows [r0,r1) of layer L the
    list of (parent layer, set of parent columns, row0, row1) it reads.  row1 None = all rows."""
    t = L["type"]
    p0, p1 = L["p0"], L["p1"]
    cols = range(c0, c1)
    if t in ("conv", "maxpool", "avgpool"):
        OH, OW, IH, IW, k, s, p = L["H"], L["W"], L["inH"], L["inW"], L["size"], L["stride"], L["pad"]
        need = set()
        for c in cols:
            b, oh, ow = c // (OH * OW), (c // OW) % OH, c % OW
            for kh in range(k):
                for kw in range(k):
                    ih, iw = oh * s - p + kh, ow * s - p + kw
                    if 0 <= ih < IH and 0 <= iw < IW:
                        need.add((b * IH + ih) * IW + iw)
        return [(p0, need, 0, None)] if t == "conv" else [(p0, need, r0, r1)]
    if t == "fc":
        hw = L["inH"] * L["inW"]
        return [(p0, {b * hw + j for b in cols for j in range(hw)}, 0, None)]
    if t == "residual":
        return [(p0, set(cols), r0, r1), (p1, set(cols), r0, r1)]
    if t == "yolo":         # column = (batch, anchor, cell): rows [anchor*R, anchor*R + R) of parent column (batch, cell)
        cells, R = L["inH"] * L["inW"], L["C"]
        A = L["inC"] // R
        out = []
        for c in cols:
            seg, cell = divmod(c, cells)
            b, a = divmod(seg, A)
            out.append((p0, {b * cells + cell}, a * R, (a + 1) * R))
        return out
    if t == "append":       # first parent upsampled by stride (all its rows), second parent at the same column
        OH, OW, st = L["H"], L["W"], L["stride"]
        IH, IW = OH // st, OW // st
        up = set()
        for c in cols:
            b, oh, ow = c // (OH * OW), (c // OW) % OH, c % OW
            up.add((b * IH + oh // st) * IW + ow // st)
        return [(p0, up, 0, None), (p1, set(cols), 0, None)]
    if t in ("matmul", "layernorm", "softmax"):
        return [(p0, set(cols), 0, None)]
    if t == "attn_k":       # column = (b, head, query); rows = keys
        Hn, hd = L["n_head"], L["n_embd"] // L["n_head"]
        out = []
        for c in cols:
            b, h, q = c // (Hn * seq), (c // seq) % Hn, c % seq
            # the first parent holds the queries (only token q is read), the second the keys (every token of b):
            # reference cfg order, parent = Query, from = Key
            out.append((p0, {b * seq + q}, h * hd, (h + 1) * hd))
        keys = {(c // (Hn * seq)) for c in cols}
        heads = {((c // seq) % Hn) for c in cols}
        for b in keys:
            for h in heads:
                out.append((p1, {b * seq + s for s in range(seq)}, h * hd, (h + 1) * hd))
        return out
    if t == "attn_v":       # column = token (b, s); rows = h*hd + d;  p0 = probabilities, p1 = values
        Hn, hd = L["n_head"], L["n_embd"] // L["n_head"]
        out = []
        for h in range(r0 // hd, (r1 - 1) // hd + 1):
            out.append((p0, {(c // seq) * Hn * seq + h * seq + c % seq for c in cols}, 0, None))
        for b in {c // seq for c in cols}:
            out.append((p1, {b * seq + s for s in range(seq)}, r0, r1))
        return out
    raise ValueError(t)


@pytest.mark.parametrize("fuse", [True, False], ids=["fused", "unfused"])
@pytest.mark.parametrize("name,min_ninst", [("custom_b3", 16), ("resnet_mini_b2", 64), ("resnet_mini_b2", 1024),
                                            ("vgg_mini_b5", 32), ("bert_mini_b2_s24", 16), ("gpt_mini_b2_s20", 256),
                                            ("yolo_mini_b2", 16), ("yolo_mini_b2", 512), ("gpt_long_b1_s272", 64)])
def test_tile_graph_against_brute_force(name, min_ninst, fuse, monkeypatch):
    if not fuse:
        monkeypatch.setenv("ASPEN_GPU_NO_FUSE", "1")
    cases = dict(H.micro_cases())
    # several query tiles per sequence, ragged against both attention tile extents (272 = 8 x 32 + 16 = 2 x 128 + 16)
    cases["gpt_long_b1_s272"] = (M.gpt2_cfg(1, 64, 2, 128), "gpt", 1, 272, 13, "token_ids")
    layers, d, n, batch, seq = make(cases[name], min_ninst)
    tl, npar, off, idx = n.graph()
    T = n.num_ninst
    infos = [n.info(l) for l in range(n.num_ldata)]
    fused_res = {i["fused_into"]: l for l, i in enumerate(infos) if i["fused_into"] >= 0}     # producer -> shortcut layer
    if fuse and any(L["type"] == "residual" for L in layers):
        assert fused_res, "shortcuts after a contraction layer should be fused"
    if not fuse:
        assert not fused_res
    for prod, res in fused_res.items():
        assert infos[res]["num_ninst"] == 0 and infos[prod]["fused_residual"] == res
        assert layers[res]["type"] == "residual" and layers[res]["p0"] == prod and layers[prod]["type"] in ("conv", "fc", "matmul")
        # the producer feeds nothing but the shortcut
        assert [l for l, L in enumerate(layers) if prod in (L["p0"], L["p1"])] == [res]
    # ---- tiles partition every out_mat; in a split-K layer the `splits` partial tiles of an output tile
    #      form a group (same range): its first member stands for the group as a parent
    owner, group_of = [], {}
    for l, i in enumerate(infos):
        own = -np.ones((i["W"], i["H"]), dtype=np.int64)
        tiles = [t for t in range(i["ninst_start"], i["ninst_start"] + i["num_ninst"])]
        assert all(tl[t] == l for t in tiles)
        ranges = {}
        for t in tiles:
            ranges.setdefault(n.tile_range(t), []).append(t)
        for (c0, c1, r0, r1), ts in ranges.items():
            assert 0 <= c0 < c1 <= i["W"] and 0 <= r0 < r1 <= i["H"]
            assert (own[c0:c1, r0:r1] == -1).all(), (name, l, "tiles overlap")
            own[c0:c1, r0:r1] = min(ts)            # the group's first member owns the region
            assert len(ts) == i["splits"] and sorted(ts) == list(range(min(ts), min(ts) + len(ts)))
            if len(ts) > 1:
                assert (min(ts) - i["ninst_start"]) % i["splits"] == 0
                for t in ts:
                    group_of[t] = min(ts)
        if i["num_ninst"]:
            assert (own >= 0).all(), (name, l, "tiles leave a gap")
        if i["fused_into"] >= 0:
            own = owner[i["fused_into"]]            # written by the producer's tiles (same geometry)
            assert own.shape == (i["W"], i["H"])
        owner.append(own)
    # ---- parents from the CSR children lists
    parents = [set() for _ in range(T)]
    for t in range(T):
        rep = group_of.get(t, t)
        if rep != t:
            # every member of a group carries the group's child list; the child counts the group once
            assert list(idx[off[t]:off[t + 1]]) == list(idx[off[rep]:off[rep + 1]])
            continue
        for c in idx[off[t]:off[t + 1]]:
            assert tl[c] > tl[t]                                     # edges point forward
            assert t not in parents[c]                               # no duplicate edges
            parents[c].add(t)
    assert [len(p) for p in parents] == list(npar)
    # ---- every tile's parents = owners of every element it reads
    partials = group_of
    for t in range(T):
        l = int(tl[t])
        L = layers[l]
        c0, c1, r0, r1 = n.tile_range(t)
        produced = lambda pp: infos[pp]["num_ninst"] > 0 or infos[pp]["fused_into"] >= 0
        # the tile that runs a fused epilogue also reads the shortcut's other operand
        shortcut_need = set()
        if l in fused_res:            # any member of a split-K group may be the one that runs the epilogue
            other = layers[fused_res[l]]["p1"]
            if produced(other):
                shortcut_need = {int(v) for v in np.unique(owner[other][c0:c1, r0:r1])}
        need = set(shortcut_need)
        regions = needed_regions(L, layers, c0, c1, r0, r1, batch, seq)
        if L["type"] == "attn_v" and layers[L["p0"]]["type"] == "attn_k" and infos[L["p0"]]["num_ninst"] == 0:
            # attention fusion (the probabilities need not be kept): the V tile computes its probability columns itself,
            # so it reads what the K-attention layer would have read for them
            K = layers[L["p0"]]
            fused = []
            for (pp, cols, ra, rb) in regions:
                if pp == L["p0"]:
                    for c in sorted(cols):
                        fused += needed_regions(K, layers, c, c + 1, 0, seq, batch, seq)
                else:
                    fused.append((pp, cols, ra, rb))
            regions = fused
        pointwise = L["type"] == "matmul" or (L["type"] == "conv" and L["size"] == 1)
        if t in partials and pointwise:
            # a partial tile of a pointwise layer reads only the parent rows (= K indices) of its K slice
            slice_ = (t - infos[l]["ninst_start"]) % infos[l]["splits"]
            k0 = slice_ * infos[l]["kiters_per_split"] * 32
            k1 = min(k0 + infos[l]["kiters_per_split"] * 32, infos[L["p0"]]["H"])
            regions = [(p, cols, k0, k1) for (p, cols, _, _) in regions]
        for (p, cols, ra, rb) in regions:
            for pp in ([L["p0"], L["p1"]] if p == "either" else [p]):
                if pp is None or not cols or not produced(pp):
                    continue
                rb_ = infos[pp]["H"] if rb is None else rb
                own = owner[pp][sorted(cols)][:, ra:rb_]
                need |= {int(v) for v in np.unique(own)}
        if L["type"] == "attn_k":
            assert need <= parents[t], (name, l, t)                 # safe: everything read is awaited
            both = set()
            for pp in (L["p0"], L["p1"]):                            # and nothing beyond the two heads' columns
                hd = L["n_embd"] // L["n_head"]
                bs = {c // (L["n_head"] * seq) for c in range(c0, c1)}
                hs = {(c // seq) % L["n_head"] for c in range(c0, c1)}
                for b in bs:
                    for h in hs:
                        both |= {int(v) for v in np.unique(owner[pp][b * seq:(b + 1) * seq, h * hd:(h + 1) * hd])}
            assert parents[t] <= both, (name, l, t)
        elif L["type"] == "append":
            # second parent exact; first parent: everything read is awaited, nothing outside the hull of its columns
            assert need <= parents[t], (name, l, t)
            up = regions[0][1]
            hull = {int(v) for v in np.unique(owner[L["p0"]][min(up):max(up) + 1, :])} if produced(L["p0"]) else set()
            exact = {int(v) for v in np.unique(owner[L["p1"]][c0:c1, :])} if produced(L["p1"]) else set()
            assert parents[t] <= hull | exact, (name, l, t)
        elif L["type"] in ("conv", "maxpool", "avgpool"):
            # the library may await the contiguous hull of the window's input columns (a superset for
            # strided windows): everything read is awaited, nothing outside the hull is
            assert need <= parents[t], (name, l, t)
            pp = L["p0"]
            if produced(pp):
                cols = set().union(*[c for (_, c, _, _) in regions])
                rr = (0, infos[pp]["H"]) if L["type"] == "conv" else (r0, r1)
                if t in partials and pointwise:
                    rr = (k0, k1)
                hull = {int(v) for v in np.unique(owner[pp][min(cols):max(cols) + 1, rr[0]:rr[1]])}
                assert parents[t] <= hull | shortcut_need, (name, l, t)
        else:
            assert parents[t] == need, (name, l, t, L["type"], sorted(parents[t]), sorted(need))
    # ---- executing by the counters runs every tile exactly once (what the device engine does: the
    #      member of a split-K group that arrives last releases the group's children)
    cnt = npar.copy().astype(np.int64)
    ready = [t for t in range(T) if cnt[t] == 0]
    ran, arrived = 0, {}
    while ready:
        t = ready.pop()
        ran += 1
        if t in group_of:
            g = group_of[t]
            arrived[g] = arrived.get(g, 0) + 1
            if arrived[g] < infos[int(tl[t])]["splits"]:
                continue
        for c in idx[off[t]:off[t + 1]]:
            cnt[c] -= 1
            assert cnt[c] >= 0
            if cnt[c] == 0:
                ready.append(int(c))
    assert ran == T and (cnt == 0).all()
    n.destroy(); d.destroy()


@pytest.mark.parametrize("name", ["gpt_mini_b2_s20", "bert_mini_b2_s24"])
def test_folded_layernorms_rewire_the_tile_graph(name, monkeypatch):
    """Layer outputs not kept: a layer norm is folded into the matmul layers behind it (and, in a post-norm block, into
    the epilogue that computes the block's shortcut).  The norm owns no tiles; a folding matmul tile waits for exactly
    the tiles that write its columns of the norm's INPUT (all rows: it gathers their statistics); the tile that
    computes a shortcut whose operand is such a norm waits for its piece of the norm's input and for the row-0 tile of
    the norm's first folding layer, which stores the statistics of those columns."""
    monkeypatch.setenv("ASPEN_GPU_NARROW_TILES", "0")        # graphs this small would take 32 x 32 tiles, which do not fold
    api.lib().aspen_keep_layer_outputs(0)
    try:
        layers, d, n, batch, seq = make(H.micro_cases()[name], 32)
        tl, npar, off, idx = n.graph()
        T = n.num_ninst
        infos = [n.info(l) for l in range(n.num_ldata)]
        norms = [l for l, L in enumerate(layers[:-1]) if L["type"] == "layernorm"]
        assert norms and all(infos[l]["num_ninst"] == 0 and infos[l]["discarded"] for l in norms)
        assert sorted(set(i["folded_norm"] for i in infos if i["folded_norm"] >= 0)) == norms
        # who writes which element: a layer's own tiles (a split-K group counts as its first member), or the tiles of the
        # contraction layer that computes a fused shortcut
        owner = {}
        for l, i in enumerate(infos):
            if i["num_ninst"] == 0:
                continue
            own = -np.ones((i["W"], i["H"]), dtype=np.int64)
            for t in range(i["ninst_start"], i["ninst_start"] + i["num_ninst"], i["splits"]):
                c0, c1, r0, r1 = n.tile_range(t)
                own[c0:c1, r0:r1] = t
            owner[l] = own
        for l, i in enumerate(infos):
            if i["fused_into"] >= 0:
                owner[l] = owner[i["fused_into"]]
        parents = [set() for _ in range(T)]
        for l, i in enumerate(infos):
            for t in range(i["ninst_start"], i["ninst_start"] + i["num_ninst"], i["splits"]):
                for c in idx[off[t]:off[t + 1]]:
                    parents[c].add(t)
        checked_matmul = checked_shortcut = 0
        for l, i in enumerate(infos):
            for t in range(i["ninst_start"], i["ninst_start"] + i["num_ninst"]):
                c0, c1, r0, r1 = n.tile_range(t)
                if i["folded_norm"] >= 0:
                    x = layers[i["folded_norm"]]["p0"]
                    need = {int(v) for v in np.unique(owner[x][c0:c1, :])} if x in owner else set()
                    assert parents[t] == need, (l, t)
                    checked_matmul += 1
                if i["fused_residual"] >= 0 and layers[i["fused_residual"]]["p1"] in norms:
                    norm = layers[i["fused_residual"]]["p1"]
                    x = layers[norm]["p0"]
                    writer = min(c for c, ci in enumerate(infos) if ci["folded_norm"] == norm)
                    need = {int(v) for v in np.unique(owner[x][c0:c1, r0:r1])} if x in owner else set()
                    need |= {int(v) for v in np.unique(owner[writer][c0:c1, 0:1])}
                    assert need <= parents[t], (l, t, sorted(need - parents[t]))
                    checked_shortcut += 1
        assert checked_matmul > 0 and (checked_shortcut > 0) == name.startswith("bert")
        # executing by the counters still runs every tile exactly once
        cnt = npar.copy().astype(np.int64)
        ready = [t for t in range(T) if cnt[t] == 0]
        ran, arrived = 0, {}
        while ready:
            t = ready.pop()
            ran += 1
            i = infos[int(tl[t])]
            if i["splits"] > 1:
                g = t - (t - i["ninst_start"]) % i["splits"]
                arrived[g] = arrived.get(g, 0) + 1
                if arrived[g] < i["splits"]:
                    continue
            for c in idx[off[t]:off[t + 1]]:
                cnt[c] -= 1
                if cnt[c] == 0:
                    ready.append(int(c))
        assert ran == T and (cnt == 0).all()
        n.destroy(); d.destroy()
    finally:
        api.lib().aspen_keep_layer_outputs(1)


def test_three_channel_first_layer_contracts_a_dense_k_axis():
    """K slices (of 32) of a network's first convolution: 3 x taps without padding for up to 64 output channels (the
    7x7 stem: 147 -> 160, five slices), taps x 4 as for every other layer beyond that."""
    def first_conv_slices(filters, size):
        cfg = f"[net]\nheight=32\nwidth=32\nchannels=3\n\n[convolutional]\nfilters={filters}\nsize={size}\nstride=1\npad=1\nactivation=relu\n\n"
        layers = M.parse_cfg(cfg)
        d = api.Dnn(cfg, None)
        n = api.Nasm(d, 2, 0, 1)
        i = n.info(1)
        n.destroy(); d.destroy()
        return i["kiters_per_split"] * i["splits"]
    assert first_conv_slices(64, 7) == 5 and first_conv_slices(16, 3) == 1 and first_conv_slices(32, 5) == 3
    assert first_conv_slices(96, 7) == 7 and first_conv_slices(128, 3) == 2


def test_layers_cut_along_k_or_resolved_through_the_table_take_the_small_tile_shape():
    """Only the 64 x 64 kernels hold split-K and k-chunk-table code: a layer cut along K, and a layer whose channel
    count is not a multiple of the K slice width (so that a slice straddles taps), get that shape whatever the tile
    count asks for; their neighbours with 32-multiple channel counts keep the large shapes."""
    import ctypes
    shp = (ctypes.c_uint32 * 13)()
    api.lib().aspen_hip_tile_shapes(shp)
    shp = list(shp)
    cfg = ("[net]\nheight=64\nwidth=64\nchannels=48\n\n"
           "[convolutional]\nfilters=128\nsize=3\nstride=1\npad=1\nactivation=relu\n\n"      # 48 channels in: table
           "[convolutional]\nfilters=128\nsize=3\nstride=1\npad=1\nactivation=relu\n\n"      # 128 channels in: stepping
           "[convolutional]\nfilters=40\nsize=1\nstride=1\npad=0\nactivation=relu\n\n"       # few rows: wide shape
           "[convolutional]\nfilters=128\nsize=1\nstride=1\npad=0\nactivation=relu\n\n")     # 40 channels in: table
    d = api.Dnn(cfg, None)
    n = api.Nasm(d, 32, 0, 1)               # one tile per layer wanted: nothing but the rules above asks for small tiles
    infos = [n.info(l) for l in range(n.num_ldata)]
    n.destroy()
    small = (shp[4], shp[5])
    assert (infos[1]["tile_H"], infos[1]["tile_W"]) == small
    assert (infos[2]["tile_H"], infos[2]["tile_W"]) == (shp[0], shp[1])
    assert (infos[3]["tile_H"], infos[3]["tile_W"]) == (shp[2], shp[3])
    assert (infos[4]["tile_H"], infos[4]["tile_W"]) == small
    assert all(i["splits"] == 1 for i in infos)
    n = api.Nasm(d, 32, 0, 8192)            # many tiles wanted: the K axis of the 3x3 layers is cut, on small tiles
    infos = [n.info(l) for l in range(n.num_ldata)]
    n.destroy(); d.destroy()
    assert infos[2]["splits"] > 1
    assert all((i["tile_H"], i["tile_W"]) == small for i in infos[1:] if i["splits"] > 1)


def test_min_ninst_raises_tile_count():
    case = H.micro_cases()["resnet_mini_b2"]
    counts = []
    for m in (1, 64, 512):
        layers, d, n, _, _ = make(case, m)
        counts.append(n.num_ninst)
        n.destroy(); d.destroy()
    assert counts[0] <= counts[1] <= counts[2] and counts[0] < counts[2]


def test_error_paths(tmp_path, capfd):
    L = api.lib()
    assert not L.apu_create_dnn(b"/nonexistent/file.cfg", None)
    bad = tmp_path / "bad.cfg"
    bad.write_text("[net]\nheight=8\nwidth=8\nchannels=3\n[bogus_layer]\nfoo=1\n")
    h = L.apu_create_dnn(str(bad).encode(), None)                    # unknown sections are reported and skipped,
    assert h                                                         # as the reference's parser does (src/darknet_parser.c:447)
    assert "Unsupported section type" in capfd.readouterr().err
    L.apu_destroy_dnn(h)
    good = tmp_path / "good.cfg"
    good.write_text(M.custom_cifar_cfg())
    # a missing or malformed weight file is reported and the dnn stays without weights, as in the
    # reference (src/apu.c apu_load_dnn_data_from_file prints and returns)
    h = L.apu_create_dnn(str(good).encode(), b"/nonexistent/weights.bin")
    assert h and "not found" in capfd.readouterr().err
    L.apu_destroy_dnn(h)
    garbage = tmp_path / "w.bin"
    garbage.write_bytes(b"not an aspen data file" * 10)
    h = L.apu_create_dnn(str(good).encode(), str(garbage).encode())
    assert h and capfd.readouterr().err != ""
    L.apu_destroy_dnn(h)
    d = api.Dnn(M.custom_cifar_cfg(), None)
    assert not L.apu_create_nasm(d.h, 0, 1)                          # min_ninst_per_ldata must be >= 1
    h = L.apu_create_nasm(d.h, 64, 0)                                # batch 0 means batch 1
    a = (api.C.c_uint * 20)()
    L.aspen_nasm_ldata_info(h, 0, a)
    assert a[3] == 32 * 32
    L.apu_destroy_nasm(h)
    assert not L.apu_create_nasm(None, 64, 1)
    t = api.Dnn(M.bert_cfg(1, 128, 2, 256), None)
    assert not L.apu_create_transformer_nasm(t.h, 64, 1, 0)          # transformer without a sequence length
    n = api.Nasm(d, 2, 0, 16)
    L.apu_destroy_dnn(d.h)                                           # refused while a nasm refers to it
    assert n.info(1)["H"] > 0
    n.destroy(); d.destroy(); t.destroy()
    capfd.readouterr()


def test_weight_file_round_trip(tmp_path, capfd):
    """ASPEN_DATA written by the model tools loads; a file missing a tensor is rejected."""
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()["custom_b3"])
    wp = str(tmp_path / "w.bin")
    M.write_aspen_data(wp, tens)
    d = api.Dnn(cfg, wp)
    d.destroy()
    capfd.readouterr()
    # a tensor whose element count does not fit its layer is reported
    broken = [(i, k, (a[:-1] if (i, k) == (tens[0][0], tens[0][1]) else a)) for (i, k, a) in tens]
    M.write_aspen_data(wp, [(i, k, np.ascontiguousarray(a).reshape(-1)) for (i, k, a) in broken])
    cfgp = tmp_path / "c.cfg"
    cfgp.write_text(cfg)
    h = api.lib().apu_create_dnn(str(cfgp).encode(), wp.encode())
    assert capfd.readouterr().err != ""
    if h:
        api.lib().apu_destroy_dnn(h)


def test_generate_nasm_without_gpu_takes_the_default(capfd):
    """apu_generate_nasm times candidates on the GPU; with num_iter 0 (and on a machine without a GPU) it
    returns the default tile policy."""
    d = api.Dnn(M.custom_cifar_cfg(), None)
    g = api.Nasm(d, 2, 0, generate_iters=0)
    ref = api.Nasm(d, 2, 0, 1536)
    assert g.num_ninst == ref.num_ninst and g.num_edges == ref.num_edges
    if not api.gpu_available():
        g2 = api.Nasm(d, 2, 0, generate_iters=3)
        assert g2.num_ninst == ref.num_ninst
        g2.destroy()
    g.destroy(); ref.destroy(); d.destroy()


def test_kernel_dividers_are_exact():
    """The kernels divide by layer constants (OH*OW, OW, tiles per row, K splits) with a multiplier and a shift that
    aspen_hip_graph_create prepares (aspen_hip_divider_for): q = (((n - t) >> 1) + t) >> shift, t = high half of
    n * multiplier.  Checked against integer division for small, large, power-of-two and odd divisors, at the
    multiples of the divisor and their neighbours and at the ends of the 32-bit range."""
    import ctypes
    import random
    L = api.lib()
    L.aspen_hip_divider_for.argtypes = [ctypes.c_uint32, ctypes.POINTER(ctypes.c_uint32)]

    def divide(n, d):
        o = (ctypes.c_uint32 * 2)()
        L.aspen_hip_divider_for(d, o)
        if o[1] & 0x80:
            return n
        t = (n * o[0]) >> 32
        return ((((n - t) & 0xffffffff) >> 1) + t) >> (o[1] & 31)

    rng = random.Random(7)
    divisors = list(range(1, 200)) + [rng.randrange(1, 1 << 31) for _ in range(500)] + \
        [12544, 3136, 784, 196, 49, 112, 56, 28, 14, 7, 224, 100352, 401408, 1605632, (1 << 31) - 1, 1 << 31, (1 << 31) + 1, (1 << 32) - 1]
    for d in divisors:
        ns = [0, 1, d - 1, d, d + 1, 2 * d - 1, 2 * d, (1 << 32) - 1, (1 << 32) - 2, 1 << 31, 123456789]
        ns += [rng.randrange(0, 1 << 32) for _ in range(40)]
        ns += [k * d + e for k in range(1, 20) for e in (-1, 0, 1)]
        for n in ns:
            if 0 <= n < (1 << 32):
                assert divide(n, d) == n // d, (n, d)
