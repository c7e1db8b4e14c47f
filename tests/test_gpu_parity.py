"""GPU parity: the HIP library (through the C ABI) against the compiled-reference fixtures and the
CPU oracle, per layer, relative L2 <= 1e-4 and identical argmax."""
import os

import numpy as np
import pytest

from aspen_amd import api, models as M
from tests import helpers as H

pytestmark = pytest.mark.gpu


# engine variants of the persistent kernel: ready queue (flag 128 forbids the ordered mode small graphs take by default)
# and ordered mode (flag 64 forces it)
QUEUE, ORDERED = 128, 64


@pytest.fixture
def engine_flags():
    """Sets the engine flags for one test (2 = count executed tiles) and restores the default afterwards."""
    def set_flags(flags):
        api.lib().aspen_hip_set_flags(2 | flags)
    yield set_flags
    api.lib().aspen_hip_set_flags(2)


@pytest.mark.parametrize("mode,flags", [(api.MODE_LAYERS, 0), (api.MODE_DATAFLOW, QUEUE), (api.MODE_DATAFLOW, ORDERED)], ids=["layers", "dataflow", "ordered"])
@pytest.mark.parametrize("name", list(H.micro_cases()))
def test_micro_nets_match_reference_fixture(gpu, engine_flags, name, mode, flags):
    """Full per-layer tensors of small nets, as produced by the compiled reference."""
    engine_flags(flags)
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()[name])
    gold = np.load(os.path.join(H.GOLDEN, f"micro_{name}.npz"))
    net = H.GpuNet(cfg, tens, batch, seq, min_ninst=8, mode=mode)
    print(f"case {name} mode {mode} tiles {net.nasm.num_ninst}", flush=True)
    net.run(x)
    try:
        for l in range(net.nasm.num_ldata):
            ref = gold[f"layer{l}"]
            got = net.layer(l)
            assert got.shape == ref.shape, (l, got.shape, ref.shape)
            err = H.rel_l2(got, ref)
            assert err <= H.REL_L2_TOL, f"layer {l} ({layers[l]['type']}): rel L2 {err:.3g}"
        assert (net.layer(net.nasm.num_ldata - 1).argmax(1) == gold[f"layer{net.nasm.num_ldata - 1}"].argmax(1)).all()
        if mode == api.MODE_DATAFLOW:
            st = net.rpool.run_stats()
            assert st == {"executed": net.nasm.num_ninst, "double_runs": 0, "aborted": 0}, st
    finally:
        net.close()


@pytest.mark.parametrize("mode,flags", [(api.MODE_LAYERS, 0), (api.MODE_DATAFLOW, QUEUE), (api.MODE_DATAFLOW, ORDERED)], ids=["layers", "dataflow", "ordered"])
@pytest.mark.parametrize("name,min_ninst", [("vgg_mini_b5", 8), ("vgg_mini_b5", 1), ("custom_b3", 8), ("resnet_mini_b2", 8)])
def test_tall_tiles_of_weight_streaming_layers_match_reference_fixture(gpu, engine_flags, monkeypatch, name, min_ninst, mode, flags):
    """Layers over at most 32 columns whose weight matrix is large take 128 x 32 tiles (the FC layers of VGG-16 at
    batch 32); here the size limit is lowered so that the small networks' FC layers take them too: cut along K and
    whole, with 128, 10 and 100 output rows."""
    monkeypatch.setenv("ASPEN_GPU_WEIGHT_STREAM_BYTES", "0")
    engine_flags(flags)
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()[name])
    gold = np.load(os.path.join(H.GOLDEN, f"micro_{name}.npz"))
    net = H.GpuNet(cfg, tens, batch, seq, min_ninst=min_ninst, mode=mode)
    tall = [l for l in range(net.nasm.num_ldata) if net.nasm.info(l)["variant"] == 4 and layers[l]["type"] in ("fc", "conv", "matmul")]
    print(f"case {name} mode {mode} tiles {net.nasm.num_ninst} tall layers {[(l, net.nasm.info(l)['splits']) for l in tall]}", flush=True)
    assert tall, "no layer took the tall shape"
    net.run(x)
    try:
        for l in range(net.nasm.num_ldata):
            err = H.rel_l2(net.layer(l), gold[f"layer{l}"])
            assert err <= H.REL_L2_TOL, f"layer {l} ({layers[l]['type']}): rel L2 {err:.3g}"
        assert (net.layer(net.nasm.num_ldata - 1).argmax(1) == gold[f"layer{net.nasm.num_ldata - 1}"].argmax(1)).all()
        if mode == api.MODE_DATAFLOW:
            st = net.rpool.run_stats()
            assert st == {"executed": net.nasm.num_ninst, "double_runs": 0, "aborted": 0}, st
    finally:
        net.close()


@pytest.mark.parametrize("loads", ["cached", "coherent", "unfused", "ordered"])
@pytest.mark.parametrize("name", list(H.micro_cases()))
def test_micro_nets_match_oracle(gpu, engine_flags, name, loads, monkeypatch):
    """Same nets against the CPU oracle (full tensors), dataflow engine with few workgroups so that
    tiles of several layers are in flight together.  The graph is re-armed and re-run with a
    DIFFERENT input each time: a tile that read a stale (cached) copy of its parent's previous
    output would not match the oracle of the new input.  Both load policies of the persistent kernel
    run: activations through the caches (the default when the layout allows it) and device-coherent;
    a third variant keeps the shortcut layers as tiles of their own instead of fusing them into the
    producing contraction tile; a fourth runs the ordered mode (tiles taken in index order and prepared
    before they are ready) instead of the ready queue."""
    from oracle import cpu
    engine_flags(ORDERED if loads == "ordered" else QUEUE)
    if loads == "coherent":
        monkeypatch.setenv("ASPEN_GPU_COHERENT_LOADS", "1")      # read when the device graph is built (first run)
    if loads == "unfused":
        monkeypatch.setenv("ASPEN_GPU_NO_FUSE", "1")             # shortcuts as tiles of their own (read when the nasm is built)
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()[name])
    inputs = [x, (x * 0.5 + 0.25).astype(np.float32), (-x).astype(np.float32), x]
    net = H.GpuNet(cfg, tens, batch, seq, min_ninst=32, mode=api.MODE_DATAFLOW, workgroups=24)
    print(f"case {name} tiles {net.nasm.num_ninst}", flush=True)
    try:
        for rep, xin in enumerate(inputs):
            outs = cpu.run_network(layers, tens, xin, batch, seq)
            net.run(xin)
            st = net.rpool.run_stats()
            assert st == {"executed": net.nasm.num_ninst, "double_runs": 0, "aborted": 0}, st
            for l in range(net.nasm.num_ldata):
                err = H.rel_l2(net.layer(l), outs[l])
                assert err <= H.REL_L2_TOL, f"run {rep} layer {l} ({layers[l]['type']}): rel L2 {err:.3g}"
    finally:
        net.close()


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["resnet_mini_b2", "bert_mini_b2_s24", "yolo_mini_b2"])
def test_launch_per_layer_reruns_match_oracle(gpu, name):
    """One launch per layer, six runs on the same graph with changing inputs, each followed by downloads of
    every layer, every one checked against the oracle; split-K layers (two launches each) included."""
    from oracle import cpu
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()[name])
    net = H.GpuNet(cfg, tens, batch, seq, min_ninst=1024, mode=api.MODE_LAYERS)
    try:
        for rep in range(6):
            xin = (x * (1.0 - 0.25 * rep) + 0.125 * rep).astype(np.float32)
            outs = cpu.run_network(layers, tens, xin, batch, seq)
            net.run(xin)
            for l in range(net.nasm.num_ldata):
                err = H.rel_l2(net.layer(l), outs[l])
                assert err <= H.REL_L2_TOL, f"run {rep} layer {l} ({layers[l]['type']}): rel L2 {err:.3g}"
    finally:
        net.close()


@pytest.mark.parametrize("mode", [api.MODE_LAYERS, api.MODE_DATAFLOW], ids=["layers", "dataflow"])
def test_every_activation_and_softmax_match_oracle(gpu, mode):
    from oracle import cpu
    cfg = H.activation_zoo_cfg()
    layers = M.parse_cfg(cfg)
    tens = M.synth_weights(layers, 21, "he")
    batch = 3
    x = M.synth_input(layers, 21, batch, 0, "token_ids")
    x = (x * 2.0 - 1.0).astype(np.float32)                 # both signs, so the negative branches are exercised
    outs = cpu.run_network(layers, tens, x, batch, 0)
    assert [L["type"] for L in layers].count("softmax") == 1 and np.allclose(outs[-1].sum(axis=1), 1.0, atol=1e-5)
    assert min(float(o.min()) for o in outs[1:6]) < 0                     # negative pre-activations did occur
    net = H.GpuNet(cfg, tens, batch, 0, min_ninst=64, mode=mode)
    try:
        net.run(x)
        for l in range(net.nasm.num_ldata):
            err = H.rel_l2(net.layer(l), outs[l])
            assert err <= H.REL_L2_TOL, f"layer {l} ({layers[l]['type']}, {layers[l].get('act')}): rel L2 {err:.3g}"
        assert np.array_equal(net.layer(net.nasm.num_ldata - 1).argmax(axis=1), outs[-1].argmax(axis=1))
    finally:
        net.close()


@pytest.mark.parametrize("mode", [api.MODE_LAYERS, api.MODE_DATAFLOW], ids=["layers", "dataflow"])
@pytest.mark.parametrize("height,width,pad", [(12, 8, 0), (11, 9, 1), (10, 8, 1), (7, 5, 0)])
def test_two_by_two_pools_with_padding_and_odd_images_match_oracle(gpu, mode, height, width, pad):
    """2x2 / stride-2 max and average pools (the window the VGG and Darknet pools use; its four inputs are
    fetched together): windows that reach over the top / left padding, over the bottom / right one, and
    images whose last row and column no window covers (reference tiled_maxpool2d / tiled_avgpool2d,
    src/tiled_kernels.c:411-498: positions outside the image are skipped, the average still divides by 4)."""
    from oracle import cpu
    cfg = (f"[net]\nheight={height}\nwidth={width}\nchannels=3\n\n"
           "[convolutional]\nfilters=40\nsize=3\nstride=1\npad=1\nactivation=linear\n\n"
           f"[maxpool]\nsize=2\nstride=2\npad={pad}\n\n"
           "[convolutional]\nfilters=24\nsize=1\nstride=1\npad=0\nactivation=linear\n\n"
           f"[avgpool]\nsize=2\nstride=2\npad={pad}\n\n"
           "[connected]\noutput=10\nactivation=linear\n\n")
    layers = M.parse_cfg(cfg)
    tens = M.synth_weights(layers, 33, "he")
    batch = 5
    x = (M.synth_input(layers, 33, batch, 0, "token_ids") * 2.0 - 1.0).astype(np.float32)
    outs = cpu.run_network(layers, tens, x, batch, 0)
    net = H.GpuNet(cfg, tens, batch, 0, min_ninst=16, mode=mode)
    try:
        net.run(x)
        for l in range(net.nasm.num_ldata):
            err = H.rel_l2(net.layer(l), outs[l])
            assert err <= H.REL_L2_TOL, f"layer {l} ({layers[l]['type']}): rel L2 {err:.3g}"
    finally:
        net.close()


@pytest.mark.parametrize("mode", [api.MODE_LAYERS, api.MODE_DATAFLOW], ids=["layers", "dataflow"])
@pytest.mark.parametrize("filters,size,stride,pad,min_ninst", [(16, 7, 2, 3, 16), (64, 3, 1, 1, 16), (64, 5, 1, 0, 2048), (96, 3, 2, 1, 16), (8, 1, 1, 0, 16)])
def test_first_layer_over_three_channels_matches_oracle(gpu, mode, filters, size, stride, pad, min_ninst):
    """A convolution over three input channels keeps its K axis dense on the device (K = 3 x taps, a chunk of four K
    positions assembled from two neighbouring pixels) when it has at most 64 output channels, and the padded layout
    otherwise: window sizes whose 3 x taps is and is not a multiple of 4, strides, padding on all four sides, all
    three tile shapes (wide, small, split along K), against the oracle's convolution; the layer behind it checks
    that nothing else of the network noticed."""
    from oracle import cpu
    cfg = ("[net]\nheight=19\nwidth=23\nchannels=3\n\n" + f"[convolutional]\nfilters={filters}\nsize={size}\nstride={stride}\npad={pad}\nactivation=leaky\n\n"
           + "[convolutional]\nfilters=24\nsize=3\nstride=1\npad=1\nactivation=relu\n\n")
    layers = M.parse_cfg(cfg)
    tens = M.synth_weights(layers, 31, "he")
    batch = 5
    x = (M.synth_input(layers, 31, batch, 0, "token_ids") * 2.0 - 1.0).astype(np.float32)
    outs = cpu.run_network(layers, tens, x, batch, 0)
    net = H.GpuNet(cfg, tens, batch, 0, min_ninst=min_ninst, mode=mode)
    try:
        net.run(x)
        dense = filters <= 64
        assert net.nasm.info(1)["kiters_per_split"] * net.nasm.info(1)["splits"] >= -(-(size * size * (3 if dense else 4)) // 32)
        for l in range(1, net.nasm.num_ldata):
            err = H.rel_l2(net.layer(l), outs[l])
            assert err <= H.REL_L2_TOL, f"layer {l}: rel L2 {err:.3g}"
    finally:
        net.close()


@pytest.mark.parametrize("mode", [api.MODE_LAYERS, api.MODE_DATAFLOW], ids=["layers", "dataflow"])
def test_channel_counts_off_the_slice_width_in_a_graph_of_large_tiles(gpu, mode):
    """Layers whose K axis goes through the k-chunk table (48 and 40 input channels: a K slice of 32 straddles taps)
    next to layers that step through their taps, in a graph wide enough for the large tile shapes: the table layers
    run on 64 x 64 tiles, their neighbours on 128 x 64 / 64 x 128, all against the oracle's convolution."""
    from oracle import cpu
    cfg = ("[net]\nheight=48\nwidth=48\nchannels=48\n\n"
           "[convolutional]\nfilters=128\nsize=3\nstride=1\npad=1\nactivation=relu\n\n"
           "[convolutional]\nfilters=128\nsize=3\nstride=1\npad=1\nactivation=leaky\n\n"
           "[convolutional]\nfilters=40\nsize=1\nstride=1\npad=0\nactivation=relu\n\n"
           "[convolutional]\nfilters=128\nsize=1\nstride=1\npad=0\nactivation=relu\n\n")
    layers = M.parse_cfg(cfg)
    tens = M.synth_weights(layers, 47, "he")
    batch = 32
    x = (M.synth_input(layers, 47, batch, 0, "token_ids") * 2.0 - 1.0).astype(np.float32)
    outs = cpu.run_network(layers, tens, x, batch, 0)
    net = H.GpuNet(cfg, tens, batch, 0, min_ninst=16, mode=mode)
    try:
        net.run(x)
        shapes = [(net.nasm.info(l)["tile_H"], net.nasm.info(l)["tile_W"]) for l in range(1, 5)]
        assert shapes[0] == (64, 64) and shapes[3] == (64, 64) and shapes[1] == (128, 64) and shapes[2] == (64, 128), shapes
        for l in range(1, net.nasm.num_ldata):
            err = H.rel_l2(net.layer(l), outs[l])
            assert err <= H.REL_L2_TOL, f"layer {l}: rel L2 {err:.3g}"
    finally:
        net.close()


@pytest.mark.parametrize("mode,flags", [(api.MODE_LAYERS, 0), (api.MODE_DATAFLOW, QUEUE), (api.MODE_DATAFLOW, ORDERED)], ids=["layers", "dataflow", "ordered"])
@pytest.mark.parametrize("min_ninst,rows_per_tile", [(2048, 512), (4096, 256), (8192, 128)])
def test_short_k_layers_take_several_row_tiles_per_workgroup(gpu, engine_flags, mode, flags, min_ninst, rows_per_tile):
    """A 1 x 1 convolution with a short K axis (64 channels in) and many output channels under the 128 x 64 shape: a
    workgroup works through two or four row tiles of its column block while the layer still has the tiles it wants;
    one such layer on its own, one with a shortcut fused into its epilogue, one with 448 rows (a last row tile that is
    only half there), all against the oracle."""
    from oracle import cpu
    engine_flags(flags)
    cfg = ("[net]\nheight=64\nwidth=64\nchannels=64\n\n"
           "[convolutional]\nfilters=512\nsize=1\nstride=1\npad=0\nactivation=relu\n\n"
           "[convolutional]\nfilters=64\nsize=1\nstride=1\npad=0\nactivation=relu\n\n"
           "[convolutional]\nfilters=512\nsize=1\nstride=1\npad=0\nactivation=linear\n\n"
           "[shortcut]\nfrom=-3\nactivation=relu\n\n"
           "[convolutional]\nfilters=96\nsize=1\nstride=1\npad=0\nactivation=relu\n\n"
           "[convolutional]\nfilters=448\nsize=1\nstride=1\npad=0\nactivation=leaky\n\n")
    layers = M.parse_cfg(cfg)
    tens = M.synth_weights(layers, 61, "he")
    batch = 32
    x = (M.synth_input(layers, 61, batch, 0, "token_ids") * 2.0 - 1.0).astype(np.float32)
    outs = cpu.run_network(layers, tens, x, batch, 0)
    net = H.GpuNet(cfg, tens, batch, 0, min_ninst=min_ninst, mode=mode)
    try:
        net.run(x)
        info = [net.nasm.info(l) for l in range(net.nasm.num_ldata)]
        assert info[1]["tile_H"] == rows_per_tile and info[3]["tile_H"] == rows_per_tile, [(i["tile_H"], i["tile_W"], i["num_ninst"]) for i in info]
        assert info[6]["tile_H"] == min(rows_per_tile, 256) or rows_per_tile == 128, [(i["tile_H"], i["tile_W"], i["num_ninst"]) for i in info]
        for l in range(1, net.nasm.num_ldata):
            err = H.rel_l2(net.layer(l), outs[l])
            assert err <= H.REL_L2_TOL, f"layer {l}: rel L2 {err:.3g}"
        if mode == api.MODE_DATAFLOW:
            assert net.rpool.run_stats() == {"executed": net.nasm.num_ninst, "double_runs": 0, "aborted": 0}
    finally:
        net.close()


@pytest.mark.parametrize("fused", [False, True], ids=["two-layers", "fused"])
@pytest.mark.parametrize("mode", [api.MODE_LAYERS, api.MODE_DATAFLOW], ids=["layers", "dataflow"])
@pytest.mark.parametrize("masked", [True, False], ids=["causal", "full"])
def test_attention_over_a_long_ragged_sequence_matches_oracle(gpu, mode, masked, fused):
    """A sequence that is a multiple of neither tile extent of the attention layers: 272 tokens = 8 x 32 + 16 queries and
    2 x 128 + 16 keys per (batch, head) (4 x 64 + 16 of either for the fused tile), with and without the causal mask,
    every layer against the oracle.  fused: layer outputs are not kept, so the V-attention tiles compute scores,
    exponentials and weighted values in one pass and the probability matrix is never written."""
    from oracle import cpu
    api.lib().aspen_keep_layer_outputs(0 if fused else 1)
    try:
        _ragged_attention(mode, masked, fused)
    finally:
        api.lib().aspen_keep_layer_outputs(1)


def _ragged_attention(mode, masked, fused):
    from oracle import cpu
    cfg = M.gpt2_cfg(2, 64, 2, 128) if masked else M.bert_cfg(2, 64, 2, 128)
    layers = M.parse_cfg(cfg)
    tens = M.synth_weights(layers, 53, "gpt")
    batch, seq = 2, 272
    x = M.synth_input(layers, 53, batch, seq, "token_ids" if masked else "embeddings")
    outs = cpu.run_network(layers, tens, x, batch, seq)
    net = H.GpuNet(cfg, tens, batch, seq, min_ninst=32, mode=mode)
    try:
        net.run(x)
        infos = [net.nasm.info(l) for l in range(net.nasm.num_ldata)]
        assert fused == any(i["fused_attention"] >= 0 for i in infos)
        for l in range(1, net.nasm.num_ldata):
            if infos[l]["discarded"]:
                with pytest.raises(RuntimeError):
                    net.layer(l)
                continue
            if infos[l]["num_ninst"] == 0 and layers[l]["type"] != "residual": continue
            err = H.rel_l2(net.layer(l), outs[l])
            assert err <= H.REL_L2_TOL, f"layer {l} ({layers[l]['type']}): rel L2 {err:.3g}"
    finally:
        net.close()


@pytest.mark.parametrize("mode,flags", [(api.MODE_LAYERS, 0), (api.MODE_DATAFLOW, QUEUE), (api.MODE_DATAFLOW, ORDERED)], ids=["layers", "dataflow", "ordered"])
@pytest.mark.parametrize("name", ["bert_mini_b2_s24", "gpt_mini_b2_s20"])
def test_fused_attention_matches_oracle(gpu, engine_flags, name, mode, flags):
    """The default setting (layer outputs not kept): a V-attention layer whose probabilities nothing else reads computes
    them in its own tiles (reference tiled_k_attention + tiled_v_attention, src/tiled_kernels.c:784-1037, in one pass).
    Every layer that is written matches the oracle, on a re-armed graph with a second input as well; the
    probability matrix is reported as not available."""
    from oracle import cpu
    engine_flags(flags)
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()[name])
    api.lib().aspen_keep_layer_outputs(0)
    try:
        net = H.GpuNet(cfg, tens, batch, seq, min_ninst=32, mode=mode)
        try:
            infos = [net.nasm.info(l) for l in range(net.nasm.num_ldata)]
            assert any(i["fused_attention"] >= 0 for i in infos)
            for xin in (x, (x * 0.5 + 0.01).astype(np.float32) if name.startswith("bert") else x[::-1].copy()):
                outs = cpu.run_network(layers, tens, xin, batch, seq)
                net.run(xin)
                for l in range(1, net.nasm.num_ldata):
                    if infos[l]["discarded"]:
                        with pytest.raises(RuntimeError):
                            net.layer(l)
                        continue
                    err = H.rel_l2(net.layer(l), outs[l])
                    assert err <= H.REL_L2_TOL, f"layer {l} ({layers[l]['type']}): rel L2 {err:.3g}"
        finally:
            net.close()
    finally:
        api.lib().aspen_keep_layer_outputs(1)


@pytest.mark.parametrize("mode,flags", [(api.MODE_LAYERS, QUEUE), (api.MODE_DATAFLOW, QUEUE), (api.MODE_DATAFLOW, ORDERED)], ids=["layers", "dataflow", "dataflow-ordered"])
@pytest.mark.parametrize("name", ["bert_mini_b2_s24", "gpt_mini_b2_s20"])
def test_folded_layernorm_matches_oracle(gpu, engine_flags, monkeypatch, name, mode, flags):
    """The default setting (layer outputs not kept): the matmul layers behind a layer norm that nothing else reads take
    the norm's input and normalise it themselves (column sums gathered in the K loop, weights with the norm's scale
    folded in): y = rstd * (W' x - mean * rowsum (W')) + b' must match W LN (x) + b (reference tiled_layernorm,
    src/tiled_kernels.c:743-782, then matmul) to the tolerance of every other layer.  BERT's norms are read by the
    block's shortcut as well: the layer that computes that shortcut in its epilogue normalises the norm's input itself,
    with the column statistics one of the folding layers has stored.  Either way the norms lose their tiles (all but a
    network's last layer).  Every layer that is written matches the oracle, on a re-armed graph with a second input as
    well."""
    from oracle import cpu
    engine_flags(flags)
    monkeypatch.setenv("ASPEN_GPU_NARROW_TILES", "0")        # graphs this small would take 32 x 32 tiles, which do not fold
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()[name])
    api.lib().aspen_keep_layer_outputs(0)
    try:
        net = H.GpuNet(cfg, tens, batch, seq, min_ninst=32, mode=mode)
        try:
            infos = [net.nasm.info(l) for l in range(net.nasm.num_ldata)]
            folded = sorted(set(i["folded_norm"] for i in infos if i["folded_norm"] >= 0))
            norms = [l for l, i in enumerate(infos[:-1]) if layers[l]["type"] == "layernorm"]
            assert folded == norms and all(infos[l]["num_ninst"] == 0 and infos[l]["discarded"] for l in norms), (folded, norms)
            for xin in (x, (x * 0.5 + 0.01).astype(np.float32) if name.startswith("bert") else x[::-1].copy()):
                outs = cpu.run_network(layers, tens, xin, batch, seq)
                net.run(xin)
                for l in range(1, net.nasm.num_ldata):
                    if infos[l]["discarded"]:
                        continue
                    err = H.rel_l2(net.layer(l), outs[l])
                    assert err <= H.REL_L2_TOL, f"layer {l} ({layers[l]['type']}): rel L2 {err:.3g}"
                assert np.array_equal(net.layer(net.nasm.num_ldata - 1).argmax(axis=-1), outs[-1].argmax(axis=-1))
        finally:
            net.close()
    finally:
        api.lib().aspen_keep_layer_outputs(1)


def test_results_in_the_callers_dimension_order(gpu):
    """dse_get_ldata_result permutes a layer's native tensor into the order the caller names (reference
    get_ldata_output, src/apu.c:227-297): matrices of a transformer are (BATCH, MAT_N, MAT_M), attention
    probabilities (BATCH, NUM_HEAD, MAT_N, MAT_M), images (BATCH, OUT_H, OUT_W, OUT_C), vectors (BATCH, OUT_C).
    Checked against numpy transpositions of the native [columns][rows] read-out."""
    import itertools
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()["bert_mini_b2_s24"])
    net = H.GpuNet(cfg, tens, batch, seq, min_ninst=64, mode=api.MODE_DATAFLOW)
    try:
        net.run(x)
        kinds = {L["type"]: i for i, L in enumerate(layers)}                  # last layer of every kind
        for t in ("matmul", "layernorm", "attn_v", "residual"):
            l = kinds[t]
            native = net.layer(l)                                            # [batch*seq][M]
            cube = native.reshape(batch, seq, native.shape[1])
            names = (api.BATCH, api.MAT_N, api.MAT_M)
            for perm in itertools.permutations(range(3)):
                got = net.nasm.layer_output(l, order=[names[p] for p in perm])
                assert np.array_equal(got, cube.transpose(perm).ravel()), (t, perm)
        l = kinds["attn_k"]
        native = net.layer(l)                                                # [batch*heads*seq][seq]
        heads = native.shape[0] // (batch * seq)
        cube = native.reshape(batch, heads, seq, seq)
        names = (api.BATCH, api.NUM_HEAD, api.MAT_N, api.MAT_M)
        for perm in ((0, 1, 2, 3), (0, 1, 3, 2), (1, 0, 2, 3), (3, 2, 1, 0)):
            got = net.nasm.layer_output(l, order=[names[p] for p in perm])
            assert np.array_equal(got, cube.transpose(perm).ravel()), perm
    finally:
        net.close()
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()["custom_b3"])
    net = H.GpuNet(cfg, tens, batch, seq, min_ninst=64, mode=api.MODE_DATAFLOW)
    try:
        net.run(x)
        l = [i for i, L in enumerate(layers) if L["type"] == "maxpool"][0]
        native = net.layer(l)
        hw = int(round((native.shape[0] // batch) ** 0.5))
        cube = native.reshape(batch, hw, hw, native.shape[1])
        names = (api.BATCH, api.OUT_H, api.OUT_W, api.OUT_C)
        for perm in ((0, 3, 1, 2), (0, 1, 2, 3), (3, 0, 2, 1)):
            got = net.nasm.layer_output(l, order=[names[p] for p in perm])
            assert np.array_equal(got, cube.transpose(perm).ravel()), perm
        l = net.nasm.num_ldata - 1                                           # connected layer: (BATCH, OUT_C)
        native = net.layer(l)
        assert np.array_equal(net.nasm.layer_output(l, order=[api.OUT_C, api.BATCH]), native.T.ravel())
        # an order that is no permutation of the layer's dimensions yields the native tensor
        assert np.array_equal(net.nasm.layer_output(l, order=[api.OUT_H, api.OUT_W]), native.ravel())
    finally:
        net.close()


@pytest.mark.parametrize("flags", [QUEUE, ORDERED, -ORDERED], ids=["queue", "ordered", "ordered-armed-by-its-tiles"])
def test_engine_rearm_many_runs(gpu, engine_flags, flags):
    """Re-arm and re-run one graph many times: every run must execute each tile exactly once, never
    stall, and reproduce the first run bit for bit (tiles are deterministic; only their order varies).
    Third variant: ordered runs WITHOUT the per-tile execution counts, which is what production runs: there no arming
    pass runs between two runs, every tile sets its own dependency counter back for the next run; different inputs
    on the way check that no run saw another run's counters or data."""
    counted = flags >= 0
    engine_flags(flags)
    if not counted:
        api.lib().aspen_hip_set_flags(ORDERED)           # no counts: runs after the first skip the arming pass
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()["gpt_mini_b2_s20"])
    net = H.GpuNet(cfg, tens, batch, seq, min_ninst=64, mode=api.MODE_DATAFLOW)
    print(f"tiles {net.nasm.num_ninst}", flush=True)
    try:
        first = None
        for rep in range(40):
            net.run(x if rep == 0 else None)
            if counted:
                st = net.rpool.run_stats()
                assert st == {"executed": net.nasm.num_ninst, "double_runs": 0, "aborted": 0}, (rep, st)
            else:
                assert net.dse.last_run_ordered()
            out = net.layer(net.nasm.num_ldata - 1)
            if first is None:
                first = out
            else:
                assert np.array_equal(first, out), f"run {rep} differs from run 0"
        if not counted:
            from oracle import cpu
            for xin in ((x * 0.5).astype(np.float32), x[::-1].copy(), x):
                want = cpu.run_network(layers, tens, xin, batch, seq)
                net.run(xin)
                for l in range(1, net.nasm.num_ldata):
                    assert H.rel_l2(net.layer(l), want[l]) <= H.REL_L2_TOL, l
            assert np.array_equal(first, net.layer(net.nasm.num_ldata - 1))
    finally:
        net.close()


def test_ordered_and_queue_runs_alternate_on_one_graph(gpu):
    """An ordered run leaves its counters armed for the next ordered run; a run on the ready queue in between leaves
    the counters both engines share at their final values.  The ordered run after it has to arm again: engines
    alternate on one graph, without per-tile counts (no arming pass of their own), and every run matches the oracle."""
    from oracle import cpu
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()["resnet_mini_b2"])
    want = cpu.run_network(layers, tens, x, batch, seq)
    net = H.GpuNet(cfg, tens, batch, seq, min_ninst=64, mode=api.MODE_DATAFLOW)
    try:
        for rep, flags in enumerate((ORDERED, ORDERED, QUEUE, ORDERED, ORDERED, QUEUE, QUEUE, ORDERED)):
            api.lib().aspen_hip_set_flags(flags)
            net.run(x if rep == 0 else None)
            assert net.dse.last_run_ordered() == (flags == ORDERED), rep
            assert net.rpool.run_stats()["aborted"] == 0, rep
            for l in range(1, net.nasm.num_ldata):
                assert H.rel_l2(net.layer(l), want[l]) <= H.REL_L2_TOL, (rep, l)
    finally:
        api.lib().aspen_hip_set_flags(0)
        net.close()


def test_queue_entries_of_earlier_runs_are_never_taken(gpu):
    """Which queue slots a run rewrites depends on its flags (hand-off, per-XCD queues) and its grid, and entries carry
    a 16-bit run tag: a slot written under one setting must not be taken for a fresh entry when the tag comes round
    again.  Runs alternate the settings for several hundred runs, then cross the tag's wrap-around; every run executes
    every tile once and reproduces the first run bit for bit."""
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()["gpt_mini_b2_s20"])
    net = H.GpuNet(cfg, tens, batch, seq, min_ninst=64, mode=api.MODE_DATAFLOW)
    L = api.lib()
    try:
        first = None
        settings = [(QUEUE, 0), (QUEUE | 16, 0), (QUEUE | 32, 256), (QUEUE, 64), (QUEUE | 32 | 16, 512), (ORDERED, 0)]

        def run_and_check(rep):
            nonlocal first
            flags, wgs = settings[rep % len(settings)]
            L.aspen_hip_set_flags(2 | flags)
            L.aspen_dse_group_set_workgroups(net.dse.h, wgs)
            net.run(x if first is None else None)
            st = net.rpool.run_stats()
            assert st == {"executed": net.nasm.num_ninst, "double_runs": 0, "aborted": 0}, (rep, flags, wgs, st)
            out = net.layer(net.nasm.num_ldata - 1)
            if first is None:
                first = out
            assert np.array_equal(first, out), f"run {rep} (flags {flags}, {wgs} workgroups) differs from run 0"

        for rep in range(300):
            run_and_check(rep)
        # one run with per-XCD queues right before the wrap, plain runs across it, the same setting again after it
        net.rpool.debug_set_epoch(65533)
        for rep in (2, 0, 5, 0, 2, 1, 4, 3):
            run_and_check(rep)
    finally:
        L.aspen_hip_set_flags(2)
        net.close()


FULL = ["resnet50_b1", "resnet50_b32", "vgg16_b32", "bert_base_b8_s128", "gpt2_b4_s512", "yolov3_b1", "yolov3_b8"]


# every configuration on the persistent kernel; the small-batch ones also as one launch per layer (what the
# default engine mode picks for a single ResNet-50 image), where split-K groups straddle XCDs
FULL_RUNS = [(n, api.MODE_DATAFLOW) for n in FULL] + [("resnet50_b1", api.MODE_LAYERS), ("yolov3_b1", api.MODE_LAYERS)]


@pytest.mark.parametrize("name,mode", FULL_RUNS, ids=[f"{n}-{'dataflow' if m == api.MODE_DATAFLOW else 'layers'}" for n, m in FULL_RUNS])
def test_full_config_matches_reference_summary(gpu, name, mode):
    """The five benchmark configurations at full size against the summaries written by the compiled
    reference: per layer sampled relative L2, norm and sum; identical argmax per image / token."""
    cfg, layers, tens, x, batch, seq = H.full_config(name)
    gold = np.load(os.path.join(H.GOLDEN, f"{name}.npz"))
    net = H.GpuNet(cfg, tens, batch, seq, min_ninst=1024 if mode == api.MODE_DATAFLOW else 128, mode=mode)
    print(f"config {name} tiles {net.nasm.num_ninst} edges {net.nasm.num_edges}", flush=True)
    try:
        net.run(x)
        if mode == api.MODE_DATAFLOW:
            st = net.rpool.run_stats()
            assert st == {"executed": net.nasm.num_ninst, "double_runs": 0, "aborted": 0}, st
        worst = H.check_against_summary(net, gold, layers, name)
        print(f"config {name}: worst sampled rel L2 {worst:.3g}", flush=True)
    finally:
        net.close()


@pytest.mark.timeout(900)
# (the two batch-16 networks on their own are the same graphs as in the co-scheduled pair, which is checked as a pair)
@pytest.mark.parametrize("workload", [w for w in M.WORKLOADS if w not in ("resnet50_b16", "vgg16_b16")])
def test_timed_graphs_match_oracle_on_whole_tensors(gpu, workload):
    """Exactly the graphs bench.py times (models.WORKLOADS: same tile counts, same engine, one ready pool for the
    co-scheduled pair), first with the library's default of not writing matrices that only a fused shortcut
    reads -- the setting the benchmark runs -- then with every matrix kept.  EVERY element of every layer is
    compared with the CPU oracle run on the same inputs (relative L2 <= 1e-4 per layer, identical argmax of
    the final layer); a single wrong tile anywhere fails its layer."""
    from oracle import cpu
    cfgs, _, _, min_ninst, engine = M.WORKLOADS[workload]
    mode = api.MODE_DATAFLOW if engine.startswith("dataflow") else api.MODE_LAYERS
    cases, want = [], []
    for name in cfgs:
        cfg, layers, tens, x, batch, seq = H.full_config(name)
        want.append(cpu.run_network(layers, tens, x, batch, seq))
        cases.append((name, cfg, layers, tens, x, batch, seq))
        print(f"oracle done: {name}", flush=True)
    try:
        for keep in (0, 1):
            api.lib().aspen_keep_layer_outputs(keep)
            pool = api.RPool()
            dse = api.DseGroup(1, mode)
            dse.set_rpool(pool)
            nets = []
            try:
                for name, cfg, layers, tens, x, batch, seq in cases:
                    net = H.GpuNet(cfg, tens, batch, seq, min_ninst=min_ninst, mode=mode)
                    net.rpool.destroy()
                    net.rpool = pool
                    if engine == "dataflow-ordered":
                        net.nasm.set_ordered(1)
                    pool.add_nasm_raw_input(net.nasm, x)
                    nets.append(net)
                print(f"{workload} keep={keep}: {sum(n.nasm.num_ninst for n in nets)} tiles", flush=True)
                dse.run()
                for net in nets:
                    dse.wait(net.nasm)
                dse.stop()
                if mode == api.MODE_DATAFLOW:
                    st = pool.run_stats()
                    assert st == {"executed": sum(n.nasm.num_ninst for n in nets), "double_runs": 0, "aborted": 0}, st
                    assert dse.last_run_ordered() or engine != "dataflow-ordered"
                worst = 0.0
                for (name, _, layers, *_), net, outs in zip(cases, nets, want):
                    dropped = 0
                    for l in range(net.nasm.num_ldata):
                        if keep == 0 and net.nasm.info(l)["discarded"]:
                            with pytest.raises(RuntimeError):
                                net.layer(l)
                            dropped += 1
                            continue
                        got = net.layer(l)
                        assert got.shape == outs[l].shape, (name, l, got.shape, outs[l].shape)
                        err = H.rel_l2(got, outs[l])
                        worst = max(worst, err)
                        assert err <= H.REL_L2_TOL, f"{name} keep={keep} layer {l} ({layers[l]['type']}): rel L2 {err:.3g}"
                    last = net.nasm.num_ldata - 1
                    assert np.array_equal(net.layer(last).argmax(axis=1), outs[last].argmax(axis=1)), f"{name}: argmax differs"
                    assert keep == 1 or dropped or not any(L["type"] in ("residual", "attn_k") for L in layers)
                print(f"{workload} keep={keep}: worst rel L2 {worst:.3g}", flush=True)
            finally:
                for net in nets:
                    net.dse.destroy()
                    net.nasm.destroy()
                    net.dnn.destroy()
                dse.destroy()
                pool.destroy()
    finally:
        api.lib().aspen_keep_layer_outputs(1)


@pytest.mark.parametrize("mode,flags", [(api.MODE_LAYERS, 0), (api.MODE_DATAFLOW, QUEUE), (api.MODE_DATAFLOW, ORDERED)], ids=["layers", "dataflow", "ordered"])
def test_two_nasms_of_one_dnn_share_a_pool(gpu, engine_flags, mode, flags, tmp_path):
    """The reference's second example runs two graphs of ONE model side by side (reference
    examples/2. vgg16_example/aspen_execute.c:38-50): both share the model's device weights, each has its own
    activations and input.  Here with different batch sizes and inputs; then one graph is destroyed and the
    pool runs on with the other."""
    from oracle import cpu
    engine_flags(flags)
    cfg, layers, tens, x3, _, _ = H.build_case(H.micro_cases()["custom_b3"])
    wp = str(tmp_path / "w.bin")
    M.write_aspen_data(wp, tens)
    dnn = api.Dnn(cfg, wp)
    x2 = (1.0 - x3[: 2 * (x3.shape[0] // 3)]).astype(np.float32)          # two images, different content
    na, nb = api.Nasm(dnn, 3, 0, 64), api.Nasm(dnn, 2, 0, 16)
    pool, dse = api.RPool(), api.DseGroup(1, mode)
    dse.set_rpool(pool)
    try:
        pool.add_nasm_raw_input(na, x3)
        pool.add_nasm_raw_input(nb, x2)
        dse.run(); dse.wait(na); dse.wait(nb); dse.stop()
        if mode == api.MODE_DATAFLOW:
            assert pool.run_stats() == {"executed": na.num_ninst + nb.num_ninst, "double_runs": 0, "aborted": 0}, pool.run_stats()
        ref_a, ref_b = cpu.run_network(layers, tens, x3, 3, 0), cpu.run_network(layers, tens, x2, 2, 0)
        for l in range(na.num_ldata):
            assert H.rel_l2(na.layer_output(l), ref_a[l]) <= H.REL_L2_TOL, ("a", l)
            assert H.rel_l2(nb.layer_output(l), ref_b[l]) <= H.REL_L2_TOL, ("b", l)
        na.destroy()                                                         # leaves the pool; the weights stay
        x2b = (x2 * 0.5).astype(np.float32)
        pool.add_nasm_raw_input(nb, x2b)
        dse.run(); dse.wait(nb); dse.stop()
        ref_b = cpu.run_network(layers, tens, x2b, 2, 0)
        for l in range(nb.num_ldata):
            assert H.rel_l2(nb.layer_output(l), ref_b[l]) <= H.REL_L2_TOL, ("b again", l)
    finally:
        dse.destroy(); pool.destroy(); nb.destroy(); dnn.destroy()


def test_co_inference_resnet50_vgg16_b16(gpu):
    """ResNet-50 batch 16 and VGG-16 batch 16 in one ready pool / one engine launch; each must equal
    its solo-run reference summary."""
    nets = []
    pool = api.RPool()
    dse = api.DseGroup(1, api.MODE_DATAFLOW)
    dse.set_rpool(pool)
    try:
        for name in ("resnet50_b16", "vgg16_b16"):
            cfg, layers, tens, x, batch, seq = H.full_config(name)
            net = H.GpuNet(cfg, tens, batch, seq)
            net.rpool.destroy()            # the shared pool replaces the private one
            net.rpool = pool
            pool.add_nasm_raw_input(net.nasm, x)
            nets.append((name, net, layers))
        print("co-inference tiles", sum(n.nasm.num_ninst for _, n, _ in nets), flush=True)
        dse.run()
        for _, net, _ in nets:
            dse.wait(net.nasm)
        dse.stop()
        # Completion is per nasm (reference src/dse.c:94-105, waiter :279-289): in a second run the wait for ResNet-50
        # (a quarter of the work) returns while the persistent kernel is still running VGG-16, and ResNet-50's result,
        # read at that moment, is already the final one.
        pool.reset_queue()
        for _, net, _ in nets:
            pool.reset_nasm(net.nasm)
        import time
        t0 = time.perf_counter()
        dse.run()
        resnet, vgg = nets[0][1].nasm, nets[1][1].nasm
        assert not dse.check(resnet)
        dse.wait(resnet)
        t_resnet = time.perf_counter() - t0
        still_running = api.lib().aspen_hip_idle() == 0
        assert dse.check(resnet)
        early = resnet.result()
        running_after_readout = api.lib().aspen_hip_idle() == 0
        dse.wait(vgg)
        t_vgg = time.perf_counter() - t0
        dse.stop()
        print(f"ResNet-50 B16 complete after {t_resnet * 1e3:.2f} ms (kernel still running: {still_running}, after the read-out: "
              f"{running_after_readout}), VGG-16 B16 after {t_vgg * 1e3:.2f} ms", flush=True)
        assert still_running, "ResNet-50's completion was only reported when the whole run was over"
        assert t_resnet < t_vgg
        assert np.array_equal(early, resnet.result()), "the result read while the kernel was running differs from the final one"
        st = pool.run_stats()
        assert st == {"executed": sum(n.nasm.num_ninst for _, n, _ in nets), "double_runs": 0, "aborted": 0}, st
        for name, net, layers in nets:
            gold = np.load(os.path.join(H.GOLDEN, f"{name}.npz"))
            H.check_against_summary(net, gold, layers, name)
    finally:
        for _, net, _ in nets:
            net.dse.destroy()
            net.nasm.destroy()
            net.dnn.destroy()
        dse.destroy()
        pool.destroy()


# ---- the flat seam on its own ---------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K,act", [(64, 64, 32, 0), (100, 37, 96, 4), (8, 300, 64, 0), (257, 129, 160, 8)])
def test_sgemm_seam_matches_oracle(gpu, M, N, K, act):
    """aspen_hip_sgemm (C-ABI, device pointers) against the oracle's packed micro-kernel."""
    from oracle import cpu
    L = api.lib()
    rng = np.random.default_rng(M * 1000 + N)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((N, K)).astype(np.float32)
    bias = rng.standard_normal(M).astype(np.float32)
    ldc = (M + 3) // 4 * 4
    want = cpu.activate(cpu.sgemm_packed(cpu.pack_weight(A), B, M, np.tile(bias, (N, 1))), act)
    dA, dB, dC, db = (L.aspen_hip_alloc(x) for x in (A.nbytes, B.nbytes, N * ldc * 4, bias.nbytes))
    assert dA and dB and dC and db
    for d, h in ((dA, A), (dB, B), (db, bias)):
        assert L.aspen_hip_h2d(d, h.ctypes.data, h.nbytes) == 0
    assert L.aspen_hip_sgemm(M, N, K, dA, K, dB, K, dC, ldc, db, act) == 0, L.aspen_hip_last_error()
    got = np.zeros((N, ldc), np.float32)
    assert L.aspen_hip_d2h(got.ctypes.data, dC, got.nbytes) == 0
    assert H.rel_l2(got[:, :M], want) <= H.REL_L2_TOL
    assert (got[:, M:] == 0).all()                      # padding rows are never written
    # argument checks fail with a message instead of launching
    assert L.aspen_hip_sgemm(M, N, K + 1, dA, K, dB, K, dC, ldc, db, act) != 0
    assert b"multiple" in L.aspen_hip_last_error()
    for d in (dA, dB, dC, db):
        L.aspen_hip_free(d)


@pytest.mark.gpu
def test_copy_kernel(gpu):
    L = api.lib()
    x = np.arange(1 << 20, dtype=np.float32)
    a, b = L.aspen_hip_alloc(x.nbytes), L.aspen_hip_alloc(x.nbytes)
    assert L.aspen_hip_h2d(a, x.ctypes.data, x.nbytes) == 0
    assert L.aspen_hip_copy(b, a, x.nbytes) == 0 and L.aspen_hip_sync() == 0
    y = np.zeros_like(x)
    assert L.aspen_hip_d2h(y.ctypes.data, b, y.nbytes) == 0
    assert np.array_equal(x, y)
    assert L.aspen_hip_copy(b, a, 24) != 0
    L.aspen_hip_free(a); L.aspen_hip_free(b)


@pytest.mark.gpu
def test_generate_nasm_times_candidates(gpu, capfd):
    """apu_generate_nasm (reference src/apu_nasm.c:601-639) on the GPU: candidates are timed, the chosen
    graph runs and matches the oracle."""
    from oracle import cpu
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()["resnet_mini_b2"])
    wp = os.path.join(os.environ.get("TMPDIR", "/tmp"), "gen_nasm_w.bin")
    M.write_aspen_data(wp, tens)
    dnn = api.Dnn(cfg, wp)
    os.unlink(wp)
    nasm = api.Nasm(dnn, batch, seq, generate_iters=2)
    out = capfd.readouterr().out
    assert out.count("sec per inference") == 9 and "selected" in out          # three candidates on three engines (ready queue, ordered, per layer)
    assert out.count("persistent kernel, ordered:") == 3 and out.count("persistent kernel, ready queue:") == 3
    pool, dse = api.RPool(), api.DseGroup(1, api.MODE_DATAFLOW)
    dse.set_rpool(pool)
    pool.add_nasm_raw_input(nasm, x)
    dse.run(); dse.wait(nasm); dse.stop()
    outs = cpu.run_network(layers, tens, x, batch, seq)
    for l in range(nasm.num_ldata):
        assert H.rel_l2(nasm.layer_output(l), outs[l]) <= H.REL_L2_TOL, l
    dse.destroy(); pool.destroy(); nasm.destroy(); dnn.destroy()


@pytest.mark.gpu
def test_model_loaded_from_reference_aspen_file_runs(gpu):
    """A .aspen file written by the compiled reference (tests/golden/tiny_ref.aspen), loaded through
    apu_load_dnn_from_file, must compute what the oracle computes from the original weights."""
    from oracle import cpu
    cfg, layers, tens, x, batch, seq = H.tiny_case()
    h = api.lib().apu_load_dnn_from_file(os.path.join(H.GOLDEN, "tiny_ref.aspen").encode())
    assert h
    dnn = api.Dnn.__new__(api.Dnn); dnn.h = h
    nasm = api.Nasm(dnn, batch, seq, 8)
    pool, dse = api.RPool(), api.DseGroup(1, api.MODE_DATAFLOW)
    dse.set_rpool(pool)
    pool.add_nasm_raw_input(nasm, x)
    dse.run(); dse.wait(nasm); dse.stop()
    outs = cpu.run_network(layers, tens, x, batch, seq)
    for l in range(nasm.num_ldata):
        assert H.rel_l2(nasm.layer_output(l), outs[l]) <= H.REL_L2_TOL, l
    dse.destroy(); pool.destroy(); nasm.destroy(); dnn.destroy()


@pytest.mark.gpu
def test_yolo_result_gathers_all_heads(gpu):
    """dse_get_ldata_result on a YOLO layer with a dimension order returns every detection head of the
    network, concatenated per image in layer order (reference src/dse.c:472-513)."""
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()["yolo_mini_b2"])
    net = H.GpuNet(cfg, tens, batch, seq, min_ninst=16)
    net.run(x)
    try:
        heads = [l for l, L in enumerate(layers) if L["type"] == "yolo"]
        mats = [net.layer(l) for l in heads]                         # [batch * boxes][rows] each
        got = net.nasm.layer_output(heads[-1], order=[api.BATCH, api.OUT_H, api.OUT_W, api.OUT_C])
        want = np.concatenate([m.reshape(batch, -1)[b] for b in range(batch) for m in mats])
        assert got.shape == want.shape and np.array_equal(got, want)
    finally:
        net.close()


@pytest.mark.gpu
def test_exported_pytorch_model_runs_like_pytorch(gpu, tmp_path):
    """Migration path of the reference's custom example (examples/3. custom_example): a PyTorch model
    exported by aspen_amd.export (batch-norm folded), its images written as the raw NCHW file that
    rpool_add_nasm reads, run on the GPU: logits within 1e-4 of PyTorch's, same argmax."""
    import torch
    from aspen_amd import export
    net, cfg, entries = H.export_example_model()
    wp, ip = str(tmp_path / "w.bin"), str(tmp_path / "in.bin")
    export.export_weights(wp, cfg, net.state_dict(), entries)
    x = torch.rand(5, 3, 16, 16)
    export.write_input_file(ip, x.numpy())
    want = net(x).detach().numpy()
    dnn = api.Dnn(cfg, wp)
    nasm = api.Nasm(dnn, 5, 0, 64)
    pool, dse = api.RPool(), api.DseGroup(1, api.MODE_DATAFLOW)
    dse.set_rpool(pool)
    api.lib().rpool_add_nasm(pool.h, nasm.h, ip.encode())
    dse.run(); dse.wait(nasm); dse.stop()
    got = nasm.result().reshape(5, -1)
    assert H.rel_l2(got, want) <= H.REL_L2_TOL
    assert (got.argmax(1) == want.argmax(1)).all()
    dse.destroy(); pool.destroy(); nasm.destroy(); dnn.destroy()


@pytest.mark.gpu
def test_default_discards_outputs_only_a_fused_shortcut_reads(gpu):
    """Default setting (what bench.py times): a contraction layer whose shortcut runs in its own epilogue does
    not write its pre-shortcut matrix.  Every other layer still matches the compiled reference's fixture,
    and asking for the discarded one is an error, not stale data."""
    name = "resnet_mini_b2"
    case = H.micro_cases()[name]
    cfg, layers, tens, x, batch, seq = H.build_case(case)
    gold = np.load(os.path.join(H.GOLDEN, f"micro_{name}.npz"))
    api.lib().aspen_keep_layer_outputs(0)
    try:
        for min_ninst in (64, 1024):          # without and with split-K
            net = H.GpuNet(cfg, tens, batch, seq, min_ninst=min_ninst)
            try:
                net.run(x)
                infos = [net.nasm.info(l) for l in range(net.nasm.num_ldata)]
                dropped = [l for l, i in enumerate(infos) if i["fused_residual"] >= 0]
                assert dropped
                for l in range(net.nasm.num_ldata):
                    if l in dropped:
                        with pytest.raises(RuntimeError):
                            net.layer(l)
                    else:
                        assert H.rel_l2(net.layer(l), gold[f"layer{l}"]) <= H.REL_L2_TOL, l
            finally:
                net.close()
    finally:
        api.lib().aspen_keep_layer_outputs(1)


@pytest.mark.gpu
@pytest.mark.parametrize("flags", [QUEUE, ORDERED], ids=["queue", "ordered"])
def test_stalled_run_is_reported_and_the_next_runs_recover(gpu, engine_flags, capfd, flags):
    """The persistent kernel's watchdog, forced from the host with a spin limit of one poll: the first
    workgroup that finds its queue slot still empty (ordered mode: its tile's dependency counter still
    positive) gives the run up, every workgroup leaves, the run reports the stall.  The following runs
    (persistent kernel, then one launch per layer, whose split-K groups count arrivals in the same counters)
    must be complete and correct again."""
    engine_flags(flags)
    name = "resnet_mini_b2"
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()[name])
    gold = np.load(os.path.join(H.GOLDEN, f"micro_{name}.npz"))
    net = H.GpuNet(cfg, tens, batch, seq, min_ninst=1024, mode=api.MODE_DATAFLOW)    # 1024: split-K layers
    try:
        assert any(net.nasm.info(l)["splits"] > 1 for l in range(net.nasm.num_ldata))
        api.lib().aspen_dse_group_set_spin_limit(net.dse.h, 1)
        net.run(x)
        st = net.rpool.run_stats()
        # (in ordered mode every tile is already held by a workgroup when the run is given up, and is run through on
        # whatever its parents have written so far: all tiles count as executed, the run is void all the same)
        assert st["aborted"] == 1 and (flags == ORDERED or st["executed"] < net.nasm.num_ninst), st
        assert "stalled" in capfd.readouterr().err
        # a run that was given up does not count as completed and hands out no results
        assert api.lib().dse_check_nasm_completion(net.nasm.h) == 0
        with pytest.raises(RuntimeError):
            net.layer(net.nasm.num_ldata - 1)
        capfd.readouterr()
        api.lib().aspen_dse_group_set_spin_limit(net.dse.h, 0)
        for mode in (api.MODE_DATAFLOW, api.MODE_LAYERS, api.MODE_DATAFLOW):
            net.dse.set_mode(mode)
            net.run(x)
            if mode == api.MODE_DATAFLOW:
                st = net.rpool.run_stats()
                assert st == {"executed": net.nasm.num_ninst, "double_runs": 0, "aborted": 0}, st
            for l in range(net.nasm.num_ldata):
                assert H.rel_l2(net.layer(l), gold[f"layer{l}"]) <= H.REL_L2_TOL, (mode, l)
    finally:
        net.close()


@pytest.mark.gpu
def test_reference_main_call_sequence(gpu, tmp_path):
    """The call sequence of the reference's main.c:60-151 through the raw C ABI (no Python wrapper objects):
    create dnn / nasm, rpool, engine group, add the input, run until completion, check completion, fetch
    the result in {BATCH, OUT_C, OUT_H, OUT_W} order; then the reset / run / wait / stop loop, reading
    the input from an NCHW file the second time; the print_* dumps and the teardown."""
    import ctypes as C
    from oracle import cpu
    L = api.lib()
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()["custom_b3"])
    cfg_path, w_path, in_path = str(tmp_path / "net.cfg"), str(tmp_path / "net.bin"), str(tmp_path / "in.bin")
    open(cfg_path, "w").write(cfg)
    M.write_aspen_data(w_path, tens)
    want = cpu.run_network(layers, tens, x, batch, seq)[-1]            # [batch][classes]
    dnn = L.apu_create_dnn(cfg_path.encode(), w_path.encode())
    assert dnn
    L.print_dnn_info(dnn, 0)
    nasm = L.apu_create_nasm(dnn, 64, batch)
    assert nasm
    L.print_nasm_info(nasm, 0, 0)
    rpool = L.rpool_init()
    dse = L.dse_group_init(8)                                           # thread count: accepted, not used
    L.dse_group_set_rpool(dse, rpool)
    xin = np.ascontiguousarray(x, dtype=np.float32)
    L.rpool_add_nasm_raw_input(rpool, nasm, xin.ctypes.data_as(C.c_void_p))
    L.print_rpool_info(rpool)
    assert L.dse_check_nasm_completion(nasm) == 0
    L.dse_group_run_until_nasm_completion(dse, nasm)
    assert L.dse_check_nasm_completion(nasm) == 1
    order = (C.c_int * 4)(api.BATCH, api.OUT_C, api.OUT_H, api.OUT_W)

    def fetch():
        out = C.c_void_p()
        n = L.dse_get_nasm_result(nasm, order, C.byref(out))
        assert n == want.size * 4
        a = np.ctypeslib.as_array(C.cast(out, C.POINTER(C.c_float)), shape=(n // 4,)).copy()
        L._free(out)
        return a.reshape(want.shape)

    assert H.rel_l2(fetch(), want) <= H.REL_L2_TOL
    # second inference: the reference's loop, input from a raw NCHW file this time
    chw = [l for l in layers if l["type"] == "input"][0]
    nchw = xin.reshape(batch, chw["H"], chw["W"], chw["C"]).transpose(0, 3, 1, 2)
    np.ascontiguousarray(nchw).tofile(in_path)
    for _ in range(2):
        L.rpool_reset_queue(rpool)
        L.apu_reset_nasm(nasm)
        L.rpool_add_nasm(rpool, nasm, in_path.encode())
        assert L.dse_check_nasm_completion(nasm) == 0
        L.dse_group_run(dse)
        L.dse_wait_for_nasm_completion(nasm)
        L.dse_group_stop(dse)
        assert H.rel_l2(fetch(), want) <= H.REL_L2_TOL
    L.aspen_flush_dynamic_memory()
    L.dse_group_destroy(dse)
    L.rpool_destroy(rpool)
    L.apu_destroy_nasm(nasm)
    L.apu_destroy_dnn(dnn)


@pytest.mark.gpu
@pytest.mark.parametrize("name,min_ninst,workgroups,flags", [("resnet_mini_b2", 1024, 0, 0), ("gpt_mini_b2_s20", 64, 16, 0), ("yolo_mini_b2", 16, 0, 0),
                                                            ("resnet50_b1", 128, 0, 0), ("bert_base_b8_s128", 192, 0, 0),
                                                            ("resnet_mini_b2", 1024, 0, 32), ("gpt_mini_b2_s20", 64, 16, 32),
                                                            ("resnet50_b1", 128, 0, 32), ("resnet_mini_b2", 1024, 0, 16),
                                                            ("resnet_mini_b2", 1024, 0, ORDERED), ("gpt_mini_b2_s20", 64, 16, ORDERED),
                                                            ("yolo_mini_b2", 16, 0, ORDERED), ("resnet50_b1", 128, 0, ORDERED)],
                         ids=lambda v: str(v))
def test_no_tile_starts_before_its_parents_have_ended(gpu, name, min_ninst, workgroups, flags):
    """The scheduler's invariant (reference src/dse.c:32-38, 311-317: a ninst runs only once all its parents are
    completed), checked from the per-tile start / end stamps of a traced run of the persistent kernel: along
    every dependency edge the child's start stamp is not earlier than the parent's end stamp, which is taken
    after the parent's stores were acknowledged.  The members of a split-K group release their children
    together, through whichever member finishes last: a child waits for the group's last end.
    flags: 0 = the ready queue, 32 = one ready queue per XCD, 16 = no parent -> child hand-off, 64 = ordered mode (no
    queue; a tile's start stamp is taken when its wait for the parents is over); the final layer must come out
    bit-identical to the default engine's in every variant (tiles do the same arithmetic wherever they run)."""
    micro = name in H.micro_cases()
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()[name]) if micro else H.full_config(name)
    expected = None
    if flags:
        api.lib().aspen_hip_set_flags(2 | QUEUE)
        plain = H.GpuNet(cfg, tens, batch, seq, min_ninst=min_ninst, mode=api.MODE_DATAFLOW, workgroups=workgroups)
        try:
            plain.run(x)
            expected = plain.nasm.layer_output(plain.nasm.num_ldata - 1).copy()
        finally:
            plain.close()
    api.lib().aspen_hip_set_flags(2 | 8 | (flags if flags & ORDERED else flags | QUEUE))
    net = H.GpuNet(cfg, tens, batch, seq, min_ninst=min_ninst, mode=api.MODE_DATAFLOW, workgroups=workgroups)
    try:
        for rep in range(2):                                     # also on a re-armed graph
            net.run(x if rep == 0 else None)
            st = net.rpool.run_stats()
            assert st == {"executed": net.nasm.num_ninst, "double_runs": 0, "aborted": 0}, st
            stamps = net.rpool.dataflow_trace().astype(np.int64)
            start, end = stamps[:, 0], stamps[:, 1].copy()
            assert (start > 0).all() and (end >= start).all()
            tile_layer, num_parents, child_off, child_idx = net.nasm.graph()
            grouped = 0
            for l in range(net.nasm.num_ldata):
                i = net.nasm.info(l)
                if i["splits"] > 1:
                    seg = end[i["ninst_start"]: i["ninst_start"] + i["num_ninst"]].reshape(-1, i["splits"])
                    seg[:] = seg.max(axis=1, keepdims=True)          # a view into `end`
                    grouped += 1
            parent_of_edge = np.repeat(np.arange(net.nasm.num_ninst), np.diff(child_off.astype(np.int64)))
            assert len(parent_of_edge) == len(child_idx) > 0
            early = start[child_idx] < end[parent_of_edge]
            assert not early.any(), (f"{int(early.sum())} of {len(early)} edges violated, first: parent "
                                     f"{parent_of_edge[early][0]} -> child {child_idx[early][0]}")
            # roots start without waiting, everything else after at least one parent
            assert (num_parents[child_idx] > 0).all()
            if expected is not None:
                assert np.array_equal(net.nasm.layer_output(net.nasm.num_ldata - 1), expected)
            print(f"{name} run {rep}: {len(child_idx)} edges hold, {grouped} split-K layers", flush=True)
    finally:
        api.lib().aspen_hip_set_flags(2)
        net.close()


@pytest.mark.gpu
@pytest.mark.parametrize("mode", [api.MODE_LAYERS, api.MODE_DATAFLOW], ids=["layers", "dataflow"])
def test_weights_reloaded_between_runs_are_used_by_the_next_run(gpu, mode, tmp_path):
    """apu_load_dnn_data_from_file on a model whose graph has already run releases the layers' device copies;
    the pool notices (the model's device generation moved), rebuilds its device graph and the next
    reset / run computes with the new weights -- checked against the oracle for both weight sets."""
    from oracle import cpu
    cfg, layers, tens, x, batch, seq = H.build_case(H.micro_cases()["resnet_mini_b2"])
    tens2 = [(i, k, (a * (0.5 if k == "WEIGHT" else -1.0)).astype(np.float32)) for i, k, a in tens]
    w2 = str(tmp_path / "w2.bin")
    M.write_aspen_data(w2, tens2)
    net = H.GpuNet(cfg, tens, batch, seq, min_ninst=256, mode=mode)
    try:
        net.run(x)
        want = cpu.run_network(layers, tens, x, batch, seq)
        for l in range(net.nasm.num_ldata):
            assert H.rel_l2(net.layer(l), want[l]) <= H.REL_L2_TOL, l
        gen = api.lib().aspen_dnn_device_generation(net.dnn.h)
        api.lib().apu_load_dnn_data_from_file(net.dnn.h, w2.encode())
        assert api.lib().aspen_dnn_device_generation(net.dnn.h) > gen
        for rep in range(2):
            net.run(x if rep == 0 else None)
            want2 = cpu.run_network(layers, tens2, x, batch, seq)
            for l in range(net.nasm.num_ldata):
                assert H.rel_l2(net.layer(l), want2[l]) <= H.REL_L2_TOL, (rep, l)
        assert H.rel_l2(want2[-1], want[-1]) > 1e-2           # the two weight sets do give different results
    finally:
        net.close()
