"""Whole-network parity: the benchmark configurations run cell by cell through the
C ABI and are compared bit-for-bit with the CPU oracle running the same description."""
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _run_both(spec, x, keep, fuse=True):
    from n2d2_amd import nets
    from oracle import cells
    net = nets.GpuNet(spec, x.shape[0], fuse=fuse)
    net.set_input(x)
    net.forward()
    want = cells.run_net(spec, x, keep=keep)
    for name in keep:
        if name in net.folded:      # a ScalingCell folded into its ElemWise consumer writes no tensor of its own
            continue
        got = net.tensors[name].to_numpy()
        w = want[name].astype(np.int64)
        assert got.shape == w.shape, name
        bad = np.count_nonzero(got != w)
        assert bad == 0, "%s: %d of %d values differ" % (name, bad, w.size)
    return net


def test_cells_with_several_inputs():
    """Convolutions that read several cells (their channels one behind the other), fused plan and cell by cell."""
    from n2d2_amd import nets
    spec = nets.branches_net()
    x = np.random.default_rng(44).integers(0, 256, size=(3, 3, 24, 24))
    keep = [l.name for l in spec.layers]
    _run_both(spec, x, keep)
    _run_both(spec, x, keep, fuse=False)


def test_lenet_config_full_batch():
    from n2d2_amd import nets
    spec = nets.lenet()
    x = np.random.default_rng(11).integers(0, 256, size=(256, 1, 32, 32))
    net = _run_both(spec, x, [l.name for l in spec.layers])
    # the three fully-connected cells are one launch
    assert [(k, [m.name for m in v]) for k, v in net.fc_chains.items()] == [("fc3", ["fc1", "fc2"])] and len(net.launched) == 5
    logits = net.tensors["fc3"].to_numpy()
    assert logits.shape == (256, 10, 1, 1) and np.abs(logits).max() > 1000
    # cell by cell, the vectors between the fully-connected cells are stored and checked too
    apart = _run_both(spec, x, [l.name for l in spec.layers], fuse=False)
    assert not apart.fc_chains and len(apart.launched) == 7


def test_stage_convolution_config_full_batch():
    """The single ResNet-18 stage convolution (64 -> 64, 3x3, 56x56) at its full batch of 64 against the oracle, and the same
    result from a replayed HIP graph that holds the graph-edge conversion of the byte planes and the forward."""
    from n2d2_amd import nets
    spec = nets.single_conv_stage()
    x = np.random.default_rng(21).integers(0, 256, size=(64,) + tuple(spec.in_shape))
    net = _run_both(spec, x, [l.name for l in spec.layers])
    want = net.tensors[spec.output].to_numpy()
    replay = net.capture(2, with_input_conversion=True)
    net.tensors[spec.output].buf.zero_()
    net.input.buf.view(64, 58, 58, 64)[:, 1:57, 1:57, :].zero_()      # (the interior: the border of zeros is written once, at creation)
    assert np.array_equal(replay().to_numpy(), want)


@pytest.mark.parametrize("variant", ["pad1", "pad0_n2d2_model", "all_signed"])
def test_resnet50_config(variant):
    from n2d2_amd import nets
    spec = nets.resnet50(pool_pad=0 if variant == "pad0_n2d2_model" else 1, unsigned_data=variant != "all_signed")
    B = 3 if variant == "pad1" else 1
    x = np.random.default_rng(12).integers(0, 256, size=(B, 3, 224, 224))
    keep = ["conv1", "pool1", "conv2.1_1x1", "conv2.1_3x3", "conv2.1_1x1_x4", "conv2.1_1x1_proj", "conv2.1_sum",
            "conv2.2_shortcut_rescale", "conv2.3_sum", "conv3.1_3x3", "conv3.4_sum", "conv4.6_sum", "conv5.1_1x1_proj",
            "conv5.3_sum", "pool", "fc"]
    print("resnet50", variant, flush=True)
    net = _run_both(spec, x, keep)
    # 12 shortcut ScalingCells folded into their sums, 16 sums folded into the convolution that feeds them
    assert "conv2.2_shortcut_rescale" in net.folded and "conv2.1_1x1_proj" in net.folded and "conv2.2_1x1_x4" in net.folded
    # ... and the first residual block (the one with a projection shortcut at full resolution) runs as one launch, which
    # takes its two middle convolutions and its expansion out of the launch list as well
    # (the kernel is written for activations in [0, 255]: the all-signed variant keeps its cells apart)
    one_launch = variant != "all_signed"
    assert list(net.bottlenecks) == (["conv2.1_sum"] if one_launch else [])
    if one_launch:
        assert [m.name for m in net.bottleneck_layers["conv2.1_sum"]] == ["conv2.1_1x1", "conv2.1_3x3", "conv2.1_1x1_x4", "conv2.1_1x1_proj"]
    # ... and the first convolution computes the max pooling behind it (its own output is never written)
    assert list(net.stem_pools) == ["pool1"] and "conv1" in net.folded
    # ... and in every other block without a projection the 3x3 convolution runs in the launch of the expansion and sum
    identity = [n for n in ("conv2.2", "conv2.3", "conv3.2", "conv3.3", "conv3.4", "conv4.2", "conv4.3", "conv4.4", "conv4.5", "conv4.6")]
    if one_launch:
        assert sorted(net.chains) == [n + "_sum" for n in identity] and all(n + "_3x3" in net.folded for n in identity)
    nfolded = (32 if one_launch else 29) + len(net.chains)
    if variant == "pad0_n2d2_model":
        assert net.tensors["pool1"].H == 55
    assert len(net.folded) == nfolded and len(net.launched) == len(spec.layers) - nfolded
    # the tensors between a 1x1 and a padded 3x3 convolution carry that padding as a border of zeros, and so does the
    # input of the block that runs as one launch
    # (the network input is stored space-to-depth with the first convolution's padding as its border)
    from n2d2_amd import capi
    assert net.input.layout == capi.S2D and net.input.halo == 2
    assert sorted(n for n, t in net.tensors.items() if t.halo and n != "input") == sorted(
        [l.name[:-3] + "1x1" for l in spec.layers if l.name.endswith("_3x3") and not (one_launch and l.name == "conv2.1_3x3")]
        + (["pool1"] if one_launch else []))
    separate = nets.GpuNet(spec, x.shape[0], bottlenecks=False, stem_pool=False, chains=False)
    separate.set_input(x)
    assert not separate.bottlenecks and not separate.chains and len(separate.folded) == 28 and len(separate.launched) == len(spec.layers) - 28
    assert np.array_equal(separate.forward().to_numpy(), net.tensors[spec.output].to_numpy())
    if variant == "pad1":
        # the library says where a whole block in one launch is the faster plan (the block with a projection); asked for
        # everywhere it is taken, the 56 x 56 blocks without one run that way too, to the same logits
        everywhere = nets.GpuNet(spec, x.shape[0], bottlenecks="all")
        everywhere.set_input(x)
        assert sorted(everywhere.bottlenecks) == ["conv2.1_sum", "conv2.2_sum", "conv2.3_sum"]
        assert everywhere.bottlenecks["conv2.1_sum"].pays(x.shape[0], 56, 56) and not everywhere.bottlenecks["conv2.2_sum"].pays(x.shape[0], 56, 56)
        assert "conv2.2_sum" not in everywhere.chains and "conv3.2_sum" in everywhere.chains
        assert np.array_equal(everywhere.forward().to_numpy(), net.tensors[spec.output].to_numpy())
        unfused = _run_both(spec, x, keep, fuse=False)
        assert not unfused.folded
        plain = nets.GpuNet(spec, x.shape[0], halo=False)
        plain.set_input(x)
        assert not any(t.halo for t in plain.tensors.values())
        assert np.array_equal(plain.forward().to_numpy(), net.tensors[spec.output].to_numpy())
    assert net.tensors["pool1"].H == (55 if variant == "pad0_n2d2_model" else 56)
    if variant == "all_signed":
        assert net.tensors["conv5.3_sum"].to_numpy().max() <= 127


def test_mobilenet_v1_config():
    from n2d2_amd import nets
    spec = nets.mobilenet_v1()
    x = np.random.default_rng(13).integers(0, 256, size=(2, 3, 224, 224))
    keep = ["conv1", "conv2_dw", "conv2_pw", "conv3_dw", "conv7_pw", "conv13_dw", "conv14_pw", "pool", "fc"]
    net = _run_both(spec, x, keep)
    # at this batch no pair is large enough for the one-launch depthwise + 1x1 kernel; asked for everywhere, it takes every
    # pair with an integer rescale on 32 bits and gives the same bytes
    assert not net.dw_pws
    fused = nets.GpuNet(spec, x.shape[0], dw_pw="all")
    fused.set_input(x)
    assert len(fused.dw_pws) >= 10 and all(d.name in fused.folded for d in fused.dw_pws.values())
    assert np.array_equal(fused.forward().to_numpy(), net.tensors[spec.output].to_numpy())
    for n in ("conv2_pw", "conv7_pw", "conv14_pw"):
        assert np.array_equal(fused.tensors[n].to_numpy(), net.tensors[n].to_numpy()), n


def test_resnet18_w4a4_config():
    from n2d2_amd import nets
    spec = nets.resnet18_w4a4()
    x = np.random.default_rng(14).integers(0, 256, size=(2, 3, 224, 224))
    keep = ["conv1", "pool1", "conv2.1_a", "conv2.1_b", "conv2.1_sum", "conv3.1_proj", "conv3.1_sum", "conv5.2_sum", "pool", "fc"]
    net = _run_both(spec, x, keep)
    assert net.tensors["conv2.1_a"].to_numpy().max() <= 15
    # every 3x3 convolution reads a tensor that carries its padding: the max pooling's output, the first convolution of
    # each block, and the seven sums that a block reads as its first convolution's input and as its sum's other input
    # (the network input is stored space-to-depth with the first convolution's padding as its border)
    from n2d2_amd import capi
    assert net.input.layout == capi.S2D and net.input.halo == 2
    assert sorted(n for n, t in net.tensors.items() if t.halo and n != "input") == sorted(
        ["pool1"] + [l.name for l in spec.layers if l.name.endswith("_a")] + [l.name for l in spec.layers if l.name.endswith("_sum")][:-1])


def test_resnet50_full_batch_properties():
    """At the benchmark size (batch 128) the oracle checks a slice; the rest is covered by batch independence:
    repeated images must give identical logits wherever they sit in the batch."""
    from n2d2_amd import nets
    from oracle import cells
    spec = nets.resnet50()
    B = 128
    rng = np.random.default_rng(15)
    base = rng.integers(0, 256, size=(8, 3, 224, 224))
    idx = rng.integers(0, 8, size=B)
    idx[:8] = np.arange(8)
    x = base[idx]
    net = nets.GpuNet(spec, B)
    net.set_input(x)
    logits = net.forward().to_numpy()[:, :, 0, 0]
    for i in range(B):
        assert np.array_equal(logits[i], logits[idx[i]]), i
    want = cells.run_net(spec, base[:2])["fc"].astype(np.int64)[:, :, 0, 0]
    assert np.array_equal(logits[:2], want)
    # a second forward over the same buffers reproduces the first
    assert np.array_equal(net.forward().to_numpy()[:, :, 0, 0], logits)
    # ... and so do twenty more, tensor by tensor on a few layers of each kind, launched back to back and replayed
    # from a graph (asynchronous LDS traffic and hand-counted waits leave no room for run-to-run differences)
    watch = ["pool1", "conv2.1_sum", "conv2.2_1x1", "conv2.3_sum", "conv3.1_3x3", "conv3.4_sum", "conv4.6_sum", "conv5.3_sum", "pool", "fc"]
    ref = {n: net.tensors[n].to_numpy() for n in watch}
    replay = net.capture()
    for it in range(20):
        (net.forward if it % 2 else replay)()
        if it % 5 == 4:
            for n in watch:
                assert np.array_equal(net.tensors[n].to_numpy(), ref[n]), (it, n)


@pytest.mark.parametrize("config", ["mobilenet_v1", "resnet18_w4a4"])
def test_batch64_configs_full_batch_properties(config):
    """MobileNet-v1 and ResNet-18 W4A4 at their benchmark size (batch 64): the oracle checks a slice, batch independence
    covers the rest (repeated images give identical logits wherever they sit), and a graph replay reproduces the launches
    tensor by tensor on a layer of each kind."""
    from n2d2_amd import nets
    from oracle import cells
    spec = getattr(nets, config)()
    B = 64
    rng = np.random.default_rng(16)
    base = rng.integers(0, 256, size=(6, 3, 224, 224))
    idx = rng.integers(0, 6, size=B)
    idx[:6] = np.arange(6)
    x = base[idx]
    net = nets.GpuNet(spec, B)
    net.set_input(x)
    logits = net.forward().to_numpy()[:, :, 0, 0]
    for i in range(B):
        assert np.array_equal(logits[i], logits[idx[i]]), i
    assert len({logits[i].tobytes() for i in range(6)}) == 6
    want = cells.run_net(spec, base[:2])["fc"].astype(np.int64)[:, :, 0, 0]
    assert np.array_equal(logits[:2], want)
    if config == "mobilenet_v1":       # the large pairs of depthwise + 1x1 convolutions run as one launch each
        assert sorted(net.dw_pws) == ["conv2_pw", "conv3_pw", "conv4_pw", "conv5_pw", "conv6_pw"]
    watch = {"mobilenet_v1": ["conv1", "conv2_dw", "conv2_pw", "conv7_dw", "conv14_pw", "pool", "fc"],
             "resnet18_w4a4": ["conv1", "pool1", "conv2.1_a", "conv2.1_sum", "conv3.1_sum", "conv5.2_sum", "pool", "fc"]}[config]
    watch = [n for n in watch if n not in net.folded]
    ref = {n: net.tensors[n].to_numpy() for n in watch}
    replay = net.capture()
    for it in range(6):
        (net.forward if it % 2 else replay)()
        if it % 3 == 2:
            for n in watch:
                assert np.array_equal(net.tensors[n].to_numpy(), ref[n]), (it, n)


def test_two_forwards_on_two_streams_agree_with_sequential_runs():
    """Handles are independent: two networks launched on two streams at once (the benchmark's two-batches-in-flight mode)
    give the bytes each gives alone."""
    import torch
    from n2d2_amd import nets
    spec = nets.resnet50(image=96)
    rng = np.random.default_rng(77)
    xs = [rng.integers(0, 256, size=(6, 3, 96, 96)) for _ in range(2)]
    gn = [nets.GpuNet(spec, 6) for _ in range(2)]
    alone = []
    for g, x in zip(gn, xs):
        g.set_input(x)
        alone.append(g.forward().to_numpy().copy())
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(2)]
    for _ in range(3):
        for g, s in zip(gn, streams):
            s.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(s):
                g.forward()
        torch.cuda.synchronize()
        for g, want in zip(gn, alone):
            assert np.array_equal(g.tensors[spec.output].to_numpy(), want)
    assert not np.array_equal(alone[0], alone[1])
