"""The C++ Frame_HIP cells end to end on the GPU: nets built from INI text through the Registrar, parameters installed
as N2D2's quantization pass leaves them, outputs read back as N2D2 float tensors and compared bit-for-bit with the CPU
oracle; the SAT / LSQ quantizer classes created through the Registrar against the oracle's formulas."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fh():
    from n2d2_amd import frame_hip
    frame_hip.set_globals(8, True, True)          # what calibNetwork sets: 8-bit export, unsigned data allowed, u8 stimuli
    yield frame_hip
    frame_hip.set_globals(0, True, False)


def _compare(fh, spec, x, keep, fusion=True):
    from oracle import cells
    net = fh.build_net(spec, x.shape[0])
    net.set_fusion(fusion)
    net.initialize()
    net.set_stimuli(x)
    net.propagate()
    want = cells.run_net(spec, x, keep=keep)
    for name in keep:
        got = net.outputs(name)
        assert got.dtype == np.float32 and got.shape == want[name].shape, name
        assert np.array_equal(got, want[name]), name
        assert net.cell_info(name)["unsigned"] == spec.unsigned[name], name
    return net


def test_lenet_through_the_registrar(fh):
    from n2d2_amd import nets
    spec = nets.lenet()
    x = np.random.default_rng(31).integers(0, 256, size=(64, 1, 32, 32))
    names = [l.name for l in spec.layers]
    # the three fully-connected cells run in the launch of the last one; the two before it are not materialised
    from n2d2_amd import capi
    net = _compare(fh, spec, x, [n for n in names if n not in ("fc1", "fc2")])
    assert net.nb_folded == 2
    with pytest.raises(fh.FrameHipError) as e:
        net.outputs("fc2")
    assert "not materialised" in str(e.value)
    with capi.launch_log() as log:
        net.propagate()
    assert log.entries[-1][0].startswith("fc_chain_kernel") and len(log.entries) == 5
    # launched apart every cell is readable, and back together the logits are the same
    net.set_fusion(False)
    net.propagate()
    assert net.nb_folded == 0
    want = cells_of(spec, x, names)
    for n in names:
        assert np.array_equal(net.outputs(n), want[n]), n
    net.set_fusion(True)
    net.propagate()
    assert net.nb_folded == 2 and np.array_equal(net.outputs("fc3"), want["fc3"])
    # new weights on a cell in the middle of the run: the cells and the plan are made again
    w = np.array(spec.layers[5].w)
    spec2 = nets.lenet()
    spec2.layers[5].w = np.roll(w, 1, axis=0)
    net.set_weights("fc2", spec2.layers[5].w.astype(np.float32))
    net.propagate()
    assert net.nb_folded == 2 and np.array_equal(net.outputs("fc3"), cells_of(spec2, x, ["fc3"])["fc3"])


def cells_of(spec, x, keep):
    from oracle import cells
    return cells.run_net(spec, x, keep=keep)


def test_resnet50_through_the_registrar(fh):
    from n2d2_amd import nets
    spec = nets.resnet50()
    x = np.random.default_rng(32).integers(0, 256, size=(2, 3, 224, 224))
    net = _compare(fh, spec, x, ["pool1", "conv2.1_sum", "conv2.2_1x1", "conv3.4_sum", "conv5.3_sum", "pool", "fc"])
    # 12 shortcut ScalingCells applied inside their sums, 16 sums computed by the 1x1 convolution before them, the first
    # convolution's max pooling computed by that convolution's launch, and the first block's other three convolutions
    # (1x1, 3x3, projection) computed by its sum's launch; in the ten blocks without a projection from conv2.2 to conv4.6 the
    # 3x3 convolution is computed by the launch of the expansion and sum
    assert net.nb_folded == 42
    with pytest.raises(fh.FrameHipError, match="not materialised"):
        net.outputs("conv3.2_3x3")
    for name in ("conv2.1_1x1", "conv2.1_3x3", "conv2.1_1x1_proj", "conv2.1_1x1_x4"):
        with pytest.raises(fh.FrameHipError, match="not materialised"):
            net.outputs(name)
    with pytest.raises(fh.FrameHipError, match="pool1 computes it on the fly"):
        net.outputs("conv1")
    # the 15 tensors between a 1x1 and a padded 3x3 convolution that are written carry that padding as a border, and so
    # does the first block's input, whose 3x3 convolution reads it through the 1x1 before
    assert net.nb_halo == 16 and net.cell_info("pool1")["halo"] == 1
    with pytest.raises(fh.FrameHipError) as e:
        net.outputs("conv2.2_shortcut_rescale")
    assert "not materialised" in str(e.value)
    # a second propagate on new stimuli reuses the prepared cells
    from oracle import cells
    x2 = np.random.default_rng(33).integers(0, 256, size=(2, 3, 224, 224))
    net.set_stimuli(x2)
    net.propagate()
    assert np.array_equal(net.outputs("fc"), cells.run_net(spec, x2)["fc"])
    # the stimuli sit on the device space-to-depth and the first launch is the kernel that reads them so, pooling included
    from n2d2_amd import capi
    with capi.launch_log() as log:
        net.propagate()
    assert log.entries[0][0].startswith("conv_s2d_kernel<4, 2, true, true, 2>") and len(log.entries) == 42
    # without fusion every cell is launched and readable
    net.set_fusion(False)
    with capi.launch_log() as log:
        net.propagate()
    assert not any(e[0].startswith("conv_s2d_kernel") for e in log.entries)
    assert net.nb_folded == 0 and net.nb_halo == 0
    keep = ["conv1", "pool1", "conv2.1_1x1", "conv2.1_3x3", "conv2.1_1x1_proj", "conv2.2_shortcut_rescale", "conv2.2_1x1_x4",
            "conv2.2_sum", "fc"]
    want = cells.run_net(spec, x2, keep=keep)
    for name in keep:
        assert np.array_equal(net.outputs(name), want[name]), name
    # and back on: the plan is made again
    net.set_fusion(True)
    net.propagate()
    assert net.nb_folded == 42 and net.nb_halo == 16 and np.array_equal(net.outputs("fc"), want["fc"])
    assert np.array_equal(net.outputs("pool1"), want["pool1"])
    assert np.array_equal(net.outputs("conv2.2_1x1"), cells.run_net(spec, x2, keep=["conv2.2_1x1"])["conv2.2_1x1"])
    # a new Scaling on a convolution that the first block's launch computes: the cell and the plan are made again.  Shifts
    # this small are outside what the block's kernel takes, so the block runs as separate launches; with the first Scaling
    # back it is one launch again
    l = {l.name: l for l in spec.layers}["conv2.1_3x3"]
    first = l.act.scaling
    for scaling, folded in (((np.asarray(first) // 2).astype(first.dtype), 39), (first, 42)):
        l.act.scaling = scaling
        net.set_scaling(l.name, l.act.mode, l.act.scaling, l.act.frac_bits, l.act.clipping)
        net.propagate()
        want = cells.run_net(spec, x2, keep=["conv2.1_3x3", "conv2.1_sum", "fc"])
        assert net.nb_folded == folded
        assert np.array_equal(net.outputs("conv2.1_sum"), want["conv2.1_sum"]) and np.array_equal(net.outputs("fc"), want["fc"])
        if folded == 29:
            assert np.array_equal(net.outputs("conv2.1_3x3"), want["conv2.1_3x3"])


def test_fusion_follows_a_scaling_change(fh):
    """Changing a folded ScalingCell's Scaling, or the sum's, rebuilds the handles and the fusion plan with them."""
    from n2d2_amd import nets
    from oracle import cells
    spec = nets.resnet50(image=64)
    x = np.random.default_rng(36).integers(0, 256, size=(2, 3, 64, 64))
    net = fh.build_net(spec, 2)
    net.initialize()
    net.set_stimuli(x)
    net.propagate()
    folded = net.nb_folded
    assert folded > 0 and np.array_equal(net.outputs("fc"), cells.run_net(spec, x)["fc"])
    by_name = {l.name: l for l in spec.layers}
    sc = by_name["conv2.2_shortcut_rescale"]
    sc.act.scaling = (np.asarray(sc.act.scaling) // 2).astype(sc.act.scaling.dtype)
    sm = by_name["conv3.1_sum"]
    sm.act.scaling = np.asarray(sm.act.scaling) + np.array([0, 1], dtype=np.asarray(sm.act.scaling).dtype)
    for l in (sc, sm):
        net.set_scaling(l.name, l.act.mode, l.act.scaling, l.act.frac_bits, l.act.clipping)
    net.propagate()
    assert net.nb_folded == folded
    assert np.array_equal(net.outputs("fc"), cells.run_net(spec, x)["fc"])


def test_mobilenet_and_w4a4_through_the_registrar(fh):
    from n2d2_amd import nets
    x = np.random.default_rng(34).integers(0, 256, size=(1, 3, 224, 224))
    _compare(fh, nets.mobilenet_v1(), x, ["conv2_dw", "conv2_pw", "conv14_pw", "fc"])
    net = _compare(fh, nets.resnet18_w4a4(), x, ["conv2.1_a", "conv2.1_sum", "conv5.2_sum", "fc"])
    # every 3x3 convolution's input carries its padding: the max pooling's output, the first convolution of each block and
    # the seven sums a convolution computes and a block reads (as its first convolution's input and as its sum's other input)
    assert net.nb_halo == 1 + 8 + 7


def test_quantized_graph_moves_between_nets_through_files(fh, tmp_path):
    """A graph quantized in one place runs in another: free parameters through N2D2's text exports, bit widths and Scalings
    through DeepNet::saveQuantization / loadQuantization; the second net is built from the INI text alone and gives the
    oracle's outputs (a ResNet-50 with every scaling mode the benchmark uses, and the float-rescaled LeNet)."""
    from n2d2_amd import nets
    from oracle import cells
    for spec, x in ((nets.resnet50(image=64), np.random.default_rng(36).integers(0, 256, size=(2, 3, 64, 64))),
                    (nets.lenet(), np.random.default_rng(37).integers(0, 256, size=(3, 1, 32, 32)))):
        first = fh.build_net(spec, x.shape[0])
        d = tmp_path / spec.name
        d.mkdir()
        for l in spec.layers:
            if l.type in ("conv", "fc"):
                first.export_free_parameters(l.name, d / (l.name + ".syntxt"))
        first.save_quantization(d)
        del first
        second = fh.Net(fh.spec_to_ini(spec, x.shape[0]))
        for l in spec.layers:
            if l.type in ("conv", "fc"):
                second.import_free_parameters(l.name, d / (l.name + ".syntxt"))
        second.load_quantization(d)
        second.initialize()
        second.set_stimuli(x)
        second.propagate()
        want = cells.run_net(spec, x, keep=[spec.output])
        assert np.array_equal(second.outputs(spec.output), want[spec.output]), spec.name


def test_depthwise_cell_from_its_connection_map(fh):
    """The number of groups comes from the connection map (Cell::getNbGroups): MobileNet's first blocks built from an INI
    without any Mapping.* key, the depthwise cells given an identity map, against the oracle."""
    from n2d2_amd import nets
    from oracle import cells
    spec = nets.mobilenet_v1(image=64)
    x = np.random.default_rng(35).integers(0, 256, size=(2, 3, 64, 64))
    ini = "\n".join(line for line in fh.spec_to_ini(spec, 2).split("\n") if not line.startswith("Mapping.NbGroups"))
    net = fh.Net(ini)
    for l in spec.layers:
        if l.type == "conv" and l.groups > 1:
            net.set_mapping(l.name, np.eye(l.groups))
    fh.install_parameters(net, spec)
    net.initialize()
    net.set_stimuli(x)
    net.propagate()
    want = cells.run_net(spec, x, keep=["conv2_dw", "conv7_dw", "fc"])
    for name in ("conv2_dw", "conv7_dw", "fc"):
        assert np.array_equal(net.outputs(name), want[name]), name


def test_grouped_convolution_cells(fh):
    """ConvCells with 2 and 4 equal groups (Mapping.NbGroups in the INI; one of them again from its connection map), a depth
    multiplier (groups = channels, twice as many outputs): every cell output against the oracle."""
    from n2d2_amd import nets
    from oracle import cells, oracle as orc
    b = nets._Builder("grouped", (8, 20, 20), 41, "SingleShift")
    t = b.conv("g2", "input", 64, 3, pad=1, groups=2)
    t = b.conv("g4", t, 64, 3, stride=2, pad=1, groups=4)
    t = b.conv("mult2", t, 128, 3, pad=1, groups=64)
    t = b.pool("pool", t, "avg", 10, 10)
    b.fc("fc", t, 10, mode="None")
    spec = b.spec
    x = np.random.default_rng(41).integers(0, 256, size=(3, 8, 20, 20))
    keep = [l.name for l in spec.layers]
    _compare(fh, spec, x, keep)
    ini = "\n".join(line for line in fh.spec_to_ini(spec, 3).split("\n") if not line.startswith("Mapping.NbGroups"))
    net = fh.Net(ini)
    for l in spec.layers:
        if l.type == "conv":
            net.set_mapping(l.name, orc.group_maps(l.w.shape[1] * l.groups, l.w.shape[0], l.groups).T)
    fh.install_parameters(net, spec)
    net.initialize()
    net.set_stimuli(x)
    net.propagate()
    want = cells.run_net(spec, x, keep=keep)
    for name in keep:
        assert np.array_equal(net.outputs(name), want[name]), name


def test_convolution_cells_with_irregular_connection_maps(fh, tmp_path):
    """ConvCells whose connection map is not a set of equal groups (what the reference evaluates connection by connection):
    overlapping connections (one hand-counted group: weights {kW, kH, C, O}, indexed by channel) and two unequal groups
    (weights {kW, kH, C / 2, O}, indexed by the count of connected channels), every output against the oracle; the cell's
    parameters survive a trip through N2D2's text files, which hold the connected kernels only."""
    from n2d2_amd import nets
    from oracle import cells
    rng = np.random.default_rng(61)
    b = nets._Builder("irregular", (8, 12, 12), 61, "SingleShift")
    t = b.conv("overlap", "input", 64, 3, pad=1)
    t = b.conv("unequal", t, 12, 3, stride=2, pad=1, groups=2)
    b.fc("fc", t, 10, mode="None")
    spec = b.spec
    m1 = (rng.random((8, 64)) < 0.5).astype(np.uint8)          # [channels, outputs]
    m1[0, :] = 1
    m1[1, 0] = 0
    m1[2, 0] = 1
    m2 = np.zeros((64, 12), dtype=np.uint8)
    m2[0:32, 0:4] = 1
    m2[32:64, 4:12] = 1
    m2[40, 5] = 0
    spec.layers[0].maps, spec.layers[1].maps = m1, m2
    x = rng.integers(0, 256, size=(3, 8, 12, 12))
    keep = [l.name for l in spec.layers]
    want = cells.run_net(spec, x, keep=keep)
    assert len(np.unique(want["unequal"])) > 20

    def check(net):
        net.initialize()
        net.set_stimuli(x)
        net.propagate()
        for name in keep:
            assert np.array_equal(net.outputs(name), want[name]), name
    net = fh.build_net(spec, 3)
    net.set_mapping("overlap", m1.T)
    net.set_mapping("unequal", m2.T)
    check(net)
    # through the text files: one line per output holding the kernels of its connected channels
    for l in spec.layers[:2]:
        net.export_free_parameters(l.name, tmp_path / (l.name + ".syntxt"))
    line = open(tmp_path / "unequal_weights.syntxt").read().split("\n")[5].split()
    assert len(line) == 31 * 9                       # output 5 misses one of its group's 32 channels
    second = fh.build_net(spec, 3)
    second.set_mapping("overlap", m1.T)
    second.set_mapping("unequal", m2.T)
    for l in spec.layers[:2]:
        second.set_weights(l.name, np.zeros_like(l.w, dtype=np.float32))
        second.import_free_parameters(l.name, tmp_path / (l.name + ".syntxt"))
    check(second)
    # a map that ties the two groups together asks for weights over every channel: the cell's {.., C / 2, O} are refused
    bad = m2.copy()
    bad[32, 0] = 1
    third = fh.build_net(spec, 3)
    third.set_mapping("unequal", bad.T)
    third.initialize()
    third.set_stimuli(x)
    with pytest.raises(fh.FrameHipError):
        third.propagate()


def test_convolution_cells_with_sub_sampling(fh):
    """ConvCells with SubSampleDims (the sums of neighbouring positions added up before the bias and the activation): a
    first-layer shape, a handful of channels and a 64-channel cell, windows that do and do not divide the positions, from INI
    text through the Registrar and through the Python planner, every output against the oracle."""
    from n2d2_amd import nets
    from oracle import cells
    b = nets._Builder("subsampled", (1, 28, 28), 71, "SingleShift")
    t = b.conv("c1", "input", 6, 5, sub=(2, 2))                 # 24 x 24 positions -> 12 x 12
    t = b.conv("c2", t, 64, 3, pad=1, sub=(3, 2))               # 12 x 12 -> 4 wide, 6 high
    t = b.conv("c3", t, 32, 3, pad=1, sub=(3, 4))               # 4 x 6 -> 2 x 2, both last windows short
    b.fc("fc", t, 10, mode="None")
    spec = b.spec
    assert [l.out_shape for l in spec.layers[:3]] == [(6, 12, 12), (64, 6, 4), (32, 2, 2)]
    assert "SubSampleDims=3 2" in fh.spec_to_ini(spec, 5)
    x = np.random.default_rng(71).integers(0, 256, size=(5, 1, 28, 28))
    keep = [l.name for l in spec.layers]
    net = _compare(fh, spec, x, keep)
    assert net.nb_folded == 0 and net.nb_halo == 0
    gnet = nets.GpuNet(spec, 5)
    gnet.set_input(x)
    gnet.forward()
    want = cells.run_net(spec, x, keep=keep)
    for name in keep:
        assert np.array_equal(gnet.tensors[name].to_numpy(), want[name].astype(np.int64)), name


MINI_MOBILENET_INI = """
$BATCH=6
$WIDTH=8
DefaultModel=Frame_HIP

[database]
Type=MNIST_IDX_Database

[sp]
SizeX=28
SizeY=28
BatchSize=${BATCH}

[sp.Transformation-1]
Type=RangeAffineTransformation
FirstOperator=Divides
FirstValue=255.0

; templates, as N2D2's model files write them
[conv_def]
Type=Conv
WeightsFiller=XavierFiller
ActivationFunction=Rectifier

[dw_def]
Mapping.ChannelsPerGroup=1

[fc_def]
Type=Fc

[stem] conv_def
Input=sp
KernelDims=3 3
NbOutputs=${WIDTH}
Padding=1
Stride=2

[dw_a] conv_def dw_def
Input=stem
KernelDims=3 3
NbOutputs=[stem]NbOutputs
Padding=1

[pw_a] conv_def
Input=dw_a
KernelDims=1 1
NbOutputs=12

[pool_a]
Input=pw_a
Type=Pool
Mapping.ChannelsPerGroup=1
PoolDims=3 3
NbOutputs=[pw_a]NbOutputs
Pooling=Max
Stride=2

[dw_b] conv_def dw_def
Input=pool_a
KernelDims=2 2
NbOutputs=[pool_a]NbOutputs

[pool_b]
Input=dw_b
Type=Pool
Mapping.ChannelsPerGroup=1
PoolDims=2 2
NbOutputs=[dw_b]NbOutputs
Pooling=Average

[fc_a] fc_def
Input=pool_b
ActivationFunction=Rectifier
NbOutputs=16

[fc_b] fc_def
Input=fc_a
ActivationFunction=Linear
NbOutputs=10

[softmax]
Input=fc_b
Type=Softmax
NbOutputs=[fc_b]NbOutputs

[softmax.Target]
"""


def test_model_file_syntax_of_the_reference(fh):
    """An INI written the way N2D2's own model files are (tests/tests_data/mnist_model/model.ini: several templates behind a
    section header, $VARIABLES, NbOutputs=[other]NbOutputs, scalar Padding / Stride, database / transformation / target sections, a
    Softmax at the end, which the integer graph does not instantiate): the cells it describes against the oracle."""
    from n2d2_amd import nets
    b = nets._Builder("mini", (1, 28, 28), 53, "SingleShift")
    t = b.conv("stem", "input", 8, 3, stride=2, pad=1)
    t = b.conv("dw_a", t, 8, 3, pad=1, groups=8)
    t = b.conv("pw_a", t, 12, 1)
    t = b.pool("pool_a", t, "max", 3, 2)
    t = b.conv("dw_b", t, 12, 2, groups=12)
    t = b.pool("pool_b", t, "avg", 2, 1)
    t = b.fc("fc_a", t, 16, kind="Rectifier")
    b.fc("fc_b", t, 10, mode="None")
    spec = b.spec
    net = fh.Net(MINI_MOBILENET_INI)
    assert net.nb_cells == len(spec.layers)           # no Softmax cell
    fh.install_parameters(net, spec)
    net.initialize()
    x = np.random.default_rng(53).integers(0, 256, size=(6, 1, 28, 28))
    net.set_stimuli(x)
    net.propagate()
    from oracle import cells
    keep = [l.name for l in spec.layers]
    want = cells.run_net(spec, x, keep=keep)
    # (fc_b computes fc_a in its own launch: read every cell with the cells launched apart, the logits both ways)
    assert net.nb_folded == 1 and np.array_equal(net.outputs("fc_b"), want["fc_b"])
    net.set_fusion(False)
    net.propagate()
    for name in keep:
        assert np.array_equal(net.outputs(name), want[name]), name
    with pytest.raises(fh.FrameHipError, match="refers to unknown section"):
        fh.Net(MINI_MOBILENET_INI.replace("[stem]NbOutputs", "[nowhere]NbOutputs"))


MULTIBRANCH_INI = """
DefaultModel=Frame_HIP

[sp]
SizeX=28
SizeY=28
BatchSize=4

[c1]
Input=sp
Type=Conv
ActivationFunction=Rectifier
KernelDims=3 3
NbOutputs=8
Stride=2

[c2]
Input=c1
Type=Conv
ActivationFunction=Rectifier
KernelDims=3 3
NbOutputs=8

; three branches with 3, 4 and 3 channels
[left1]
Input=c2
Type=Conv
ActivationFunction=Rectifier
KernelDims=3 3
NbOutputs=3

[left2]
Input=left1
Type=Conv
ActivationFunction=Rectifier
KernelDims=3 3
NbOutputs=3
Padding=1

[mid1]
Input=c2
Type=Conv
ActivationFunction=Rectifier
KernelDims=2 2
NbOutputs=4

[mid2]
Input=mid1
Type=Conv
ActivationFunction=Rectifier
KernelDims=2 2
NbOutputs=4

[right1]
Input=c2
Type=Conv
ActivationFunction=Rectifier
KernelDims=3 3
NbOutputs=3

; the convolution that reads all three
[join]
Input=left2,mid2,right1
Type=Conv
ActivationFunction=Rectifier
KernelDims=3 3
NbOutputs=10

[after]
Input=join
Type=Conv
ActivationFunction=Rectifier
KernelDims=3 3
NbOutputs=[join]NbOutputs
Padding=1

[sum]
Input=join,after
Type=ElemWise
NbOutputs=[after]NbOutputs
Operation=Sum
ActivationFunction=Linear
Weights=1 2
Shifts=0 3

[head]
Input=sum
Type=Conv
ActivationFunction=Linear
KernelDims=7 7
NbOutputs=10

[softmax]
Input=head
Type=Softmax
NbOutputs=[head]NbOutputs
"""


def test_a_multibranch_model_file(fh):
    """The shape of the reference's multi-branch fixture (tests/tests_data/mnist_multibranch_model/model.ini): branches of 3
    and 4 channels, a convolution that reads three cells, a sum of two cells, a Softmax at the end; every cell against the
    oracle, with and without the fusion plan."""
    from n2d2_amd import nets
    from oracle import cells
    b = nets._Builder("multibranch", (1, 28, 28), 59, "SingleShift")
    t = b.conv("c1", "input", 8, 3, stride=2)
    c2 = b.conv("c2", t, 8, 3)
    l = b.conv("left2", b.conv("left1", c2, 3, 3), 3, 3, pad=1)
    m = b.conv("mid2", b.conv("mid1", c2, 4, 2), 4, 2)
    r = b.conv("right1", c2, 3, 3)
    j = b.conv("join", [l, m, r], 10, 3)
    a = b.conv("after", j, 10, 3, pad=1)
    s_ = b.sum("sum", [j, a], kind="Linear", weights=[1, 2], shifts=[0, 3])
    b.conv("head", s_, 10, 7, kind="Linear")
    spec = b.spec
    x = np.random.default_rng(59).integers(0, 256, size=(4, 1, 28, 28))
    keep = [l_.name for l_ in spec.layers]
    want = cells.run_net(spec, x, keep=keep)
    for fusion in (True, False):
        net = fh.Net(MULTIBRANCH_INI)
        assert net.nb_cells == len(spec.layers)
        fh.install_parameters(net, spec)
        net.set_fusion(fusion)
        net.initialize()
        net.set_stimuli(x)
        net.propagate()
        for name in keep:
            assert np.array_equal(net.outputs(name), want[name]), (name, fusion)


POOL_MAPPINGS_INI = """
[p_full]
Input=c1
Type=Pool
PoolDims=2 2
Stride=2
NbOutputs=2
Pooling=Max

[p_groups]
Input=c1
Type=Pool
PoolDims=3 3
Stride=2
NbOutputs=3
Pooling=Average
Mapping.NbGroups=3

[p_step]
Input=c1
Type=Pool
PoolDims=2 2
Stride=2
NbOutputs=3
Pooling=Max
Mapping.SizeY=3
Mapping.StrideY=2
Mapping.OffsetY=1

[p_hand]
Input=c1
Type=Pool
PoolDims=3 3
Stride=1
Padding=1
NbOutputs=2
Pooling=Average
Mapping(c1)=1 0  0 1  1 1  0 0  0 1  1 0

[p_two]
Input=c1,c2
Type=Pool
PoolDims=2 2
Stride=2
NbOutputs=2
Pooling=Max
Mapping(c1).SizeY=0
Mapping(c1).NbIterations=1
Mapping(c2).SizeY=0
Mapping(c2).NbIterations=1
Mapping(c2).OffsetX=1
"""


def test_pool_cells_with_connection_maps(fh):
    """Pool sections with the Mapping keys of src/Generator/MappingGenerator.cpp:33-201: none (every channel behind every
    output), equal groups, a patch stepped along the diagonal, a matrix written out, and two parents with a map each; the
    maps expected here are written down by hand from that file's loops, the outputs come from the oracle's pooling with them."""
    from n2d2_amd import nets
    from oracle import cells
    b = nets._Builder("maps", (1, 14, 14), 83, "SingleShift")
    b.conv("c1", "input", 6, 3)
    b.conv("c2", "input", 6, 3)
    spec = b.spec
    x = np.random.default_rng(83).integers(0, 256, size=(3, 1, 14, 14))
    want = cells.run_net(spec, x, keep=["c1", "c2"])
    net = fh.Net(fh.spec_to_ini(spec, 3) + POOL_MAPPINGS_INI)
    fh.install_parameters(net, spec)
    net.initialize()
    net.set_stimuli(x)
    net.propagate()
    c1, c2 = net.outputs("c1"), net.outputs("c2")
    assert np.array_equal(c1, want["c1"]) and np.array_equal(c2, want["c2"])

    def m(rows):            # [channel][output]
        return np.array(rows, dtype=np.uint8)
    full = np.ones((6, 2), dtype=np.uint8)
    groups = m([[1, 0, 0], [1, 0, 0], [0, 1, 0], [0, 1, 0], [0, 0, 1], [0, 0, 1]])
    # x = i, y = 1 + 2 i for i = 0..5, a patch of 1 output x 3 channels, both modulo the sizes
    step = m([[0, 0, 1], [1, 0, 1], [1, 0, 0], [1, 1, 0], [0, 1, 0], [0, 1, 1]])
    hand = m([[1, 0], [0, 1], [1, 1], [0, 0], [0, 1], [1, 0]])
    # one iteration each: output 0 pools all of c1, output 1 all of c2
    two = m([[1, 0]] * 6 + [[0, 1]] * 6)
    for name, kind, pool, stride, pad, maps, src in (("p_full", "max", 2, 2, 0, full, c1), ("p_groups", "avg", 3, 2, 0, groups, c1),
                                                    ("p_step", "max", 2, 2, 0, step, c1), ("p_hand", "avg", 3, 1, 1, hand, c1),
                                                    ("p_two", "max", 2, 2, 0, two, np.concatenate([c1, c2], 1))):
        ref = cells.pool_cell(src, kind, (pool, pool), (stride, stride), (pad, pad), maps=maps)
        assert np.array_equal(net.outputs(name), ref), name
    # A map set after initialize() is used by the next propagate (it is not silently ignored), also where the cell has as
    # many outputs as channels, and a map of the wrong size is refused
    b2 = nets._Builder("late", (1, 14, 14), 84, "SingleShift")
    t = b2.conv("c1", "input", 6, 3)
    b2.pool("p", t, "max", 2, 2)
    spec2 = b2.spec
    net2 = fh.Net(fh.spec_to_ini(spec2, 3))
    fh.install_parameters(net2, spec2)
    net2.initialize()
    net2.set_stimuli(x)
    net2.propagate()
    c1 = net2.outputs("c1")
    assert np.array_equal(net2.outputs("p"), cells.pool_cell(c1, "max", (2, 2), (2, 2), (0, 0)))
    late = np.roll(np.eye(6, dtype=np.uint8), 1, axis=1) | np.eye(6, dtype=np.uint8)        # [channel][output]: outputs pool two channels
    net2.set_mapping("p", late.T)
    net2.propagate()
    assert np.array_equal(net2.outputs("p"), cells.pool_cell(c1, "max", (2, 2), (2, 2), (0, 0), maps=late))
    with pytest.raises(RuntimeError, match="nbOutputs, nbChannels"):
        net2.set_mapping("p", np.ones((6, 5)))


def test_cells_with_two_outputs_through_the_registrar(fh):
    """A binary classifier: a convolution with 3 outputs, a rescaled FC with 2 and a last FC with 2 raw logits (output
    tensors whose pixel is one dword), through the Registrar cells and through GpuNet."""
    from n2d2_amd import nets
    b = nets._Builder("binary", (3, 16, 16), 47, "SingleShift")
    t = b.conv("c1", "input", 16, 3, stride=2, pad=1)
    t = b.conv("c2", t, 3, 3, pad=1)
    t = b.pool("pool", t, "max", 2, 2)
    t = b.fc("fc1", t, 2, kind="Rectifier")
    b.fc("fc2", t, 2, mode="None")
    spec = b.spec
    x = np.random.default_rng(47).integers(0, 256, size=(5, 3, 16, 16))
    keep = [l.name for l in spec.layers]
    _compare(fh, spec, x, keep)
    from oracle import cells
    g = nets.GpuNet(spec, 5)
    g.set_input(x)
    g.forward()
    want = cells.run_net(spec, x, keep=keep)
    for name in keep:
        if name not in g.folded:
            assert np.array_equal(g.tensors[name].to_numpy(), want[name].astype(np.int64)), name


def test_convolution_cells_with_several_inputs(fh):
    """Cells whose Input lists several cells see those cells' channels one behind the other (src/Cell/ConvCell_Frame.cpp:
    438-459): two such ConvCells, one of them feeding a sum, an average and a max PoolCell over two cells each, and an
    FcCell with two inputs (the bias once per input, src/Cell/FcCell_Frame.cpp:309), through the Registrar cells with and without the fusion plan (a cell with several
    inputs keeps its own launch), every output against the oracle."""
    from n2d2_amd import nets
    spec = nets.branches_net()
    x = np.random.default_rng(43).integers(0, 256, size=(3, 3, 24, 24))
    keep = [l.name for l in spec.layers]
    net = _compare(fh, spec, x, keep, fusion=False)
    net.set_fusion(True)
    net.propagate()
    from oracle import cells
    want = cells.run_net(spec, x, keep=["join", "sum", "fc"])
    for name in ("join", "sum", "fc"):
        assert np.array_equal(net.outputs(name), want[name]), name


def test_depthwise_and_pointwise_cells_run_as_one_launch(fh):
    """DeepNet::planFusion gives a 3x3 depthwise ConvCell to the 1x1 ConvCell that alone reads it where the pair is large
    enough: MobileNet at 256 x 256, batch 8 (blocks 2 to 4); same logits as the oracle and as the cells launched apart,
    and the depthwise outputs are not there to read."""
    from n2d2_amd import nets
    from oracle import cells
    spec = nets.mobilenet_v1(image=256)
    x = np.random.default_rng(36).integers(0, 256, size=(8, 3, 256, 256))
    net = fh.build_net(spec, 8)
    net.initialize()
    net.set_stimuli(x)
    net.propagate()
    want = cells.run_net(spec, x[:2], keep=["conv2_pw", "conv4_pw", "fc"])
    assert net.nb_folded == 3
    for name in ("conv2_pw", "conv4_pw", "fc"):
        assert np.array_equal(net.outputs(name)[:2], want[name]), name
    with pytest.raises(fh.FrameHipError) as e:
        net.outputs("conv3_dw")
    assert "not materialised" in str(e.value)
    fused_logits = net.outputs("fc").copy()
    net.set_fusion(False)
    net.propagate()
    assert net.nb_folded == 0
    assert np.array_equal(net.outputs("fc"), fused_logits)
    assert np.array_equal(net.outputs("conv3_dw")[:2], cells.run_net(spec, x[:2], keep=["conv3_dw"])["conv3_dw"])


def test_signedness_change_rebuilds_the_cells(fh):
    """-no-unsigned (DeepNetExport::mUnsignedData = false): every cell saturates to the signed range."""
    from n2d2_amd import nets
    from oracle import cells
    spec_u = nets.resnet50(image=64)
    spec_s = nets.resnet50(image=64, unsigned_data=False)
    x = np.random.default_rng(35).integers(0, 128, size=(1, 3, 64, 64))
    try:
        fh.set_globals(8, False, False)
        net = fh.build_net(spec_s, 1)
        net.initialize()
        net.set_stimuli(x)
        net.propagate()
        assert np.array_equal(net.outputs("fc"), cells.run_net(spec_s, x)["fc"])
        assert net.outputs("conv2.1_sum").max() <= 127
    finally:
        fh.set_globals(8, True, True)
    assert spec_u.unsigned["conv1"] and not spec_s.unsigned["conv1"]


def test_non_integer_weights_are_refused(fh):
    from n2d2_amd import nets
    spec = nets.lenet()
    net = fh.build_net(spec, 4)
    net.set_weights("conv1", spec.layers[0].w.astype(np.float32) + 0.25)
    net.initialize()
    net.set_stimuli(np.zeros((4, 1, 32, 32)))
    with pytest.raises(fh.FrameHipError) as e:
        net.propagate()
    assert "is not an integer" in str(e.value)


# ------------------------------------------------------------ quantizer classes

def test_sat_quantizer_cell_class(fh):
    from oracle import oracle as orc
    rng = np.random.default_rng(41)
    w = rng.normal(0, 0.05, size=64 * 64 * 9).astype(np.float32)
    g = rng.normal(size=w.size).astype(np.float32)
    for quant_mode, name in ((1, "symrange"), (0, "default"), (3, "fullrange"), (2, "asymrange")):       # QuantizerCell::QuantMode order
        wq, dw, stats = np.empty_like(w), np.empty_like(w), np.zeros(2, dtype=np.float32)
        rc = fh.lib.fh_sat_cell_run(b"Frame_HIP", w.ctypes.data, g.ctypes.data, w.size, 64 * 9, 15, quant_mode, 1, 0,
                                    wq.ctypes.data, dw.ctypes.data, stats.ctypes.data)
        assert rc == 0, fh.lib.fh_last_error()
        want, tmax, _ = orc.sat_weight_forward(w, 15.0, name)
        assert abs(stats[0] - tmax) <= 1e-5 * tmax and stats[1] == 1.0
        bad = np.abs(wq - want) > 1e-5
        assert bad.sum() <= max(2, int(2e-4 * w.size))
        want_b = orc.sat_weight_backward(g, w, 15.0, np.float32(tmax), name if name in ("fullrange", "asymrange") else "default")
        assert np.all(np.abs(dw - want_b) <= 1e-5 * np.maximum(np.abs(want_b), 1e-2))
    # ApplyScaling with outputsSize = dimB*dimY*dimX
    wq, dw, stats = np.empty_like(w), np.empty_like(w), np.zeros(2, dtype=np.float32)
    assert fh.lib.fh_sat_cell_run(b"Frame_HIP", w.ctypes.data, g.ctypes.data, w.size, 64 * 9, 15, 1, 1, 1, wq.ctypes.data, dw.ctypes.data,
                                  stats.ctypes.data) == 0
    want, tmax, scal = orc.sat_weight_forward(w.astype(np.float64), 15.0, "symrange", apply_scaling=True, outputs_size=64 * 9)
    assert abs(stats[1] - scal) <= 1e-5 * scal
    assert (np.abs(wq - want) > 1e-5 * np.abs(want).max()).sum() <= 8
    assert fh.lib.fh_sat_cell_run(b"Frame", w.ctypes.data, g.ctypes.data, w.size, 1, 15, 1, 1, 0, wq.ctypes.data, dw.ctypes.data,
                                  stats.ctypes.data) == 1                      # unknown model key


def test_sat_quantizer_activation_class_with_solver(fh):
    from oracle import oracle as orc
    rng = np.random.default_rng(42)
    n = 32 * 28 * 28
    x = rng.normal(2.0, 3.0, size=n).astype(np.float32)
    g = rng.normal(size=n).astype(np.float32)
    y, dx, alphas = np.empty_like(x), np.empty_like(x), np.zeros(3, dtype=np.float32)
    lr = 1e-4
    assert fh.lib.fh_sat_act_run(b"Frame_HIP", x.ctypes.data, g.ctypes.data, n, 15, 6.0, lr, y.ctypes.data, dx.ctypes.data, alphas.ctypes.data) == 0
    want_y, fp = orc.sat_act_forward(x, 15.0, 6.0, inference=False)
    assert (np.abs(y - want_y) > 6e-5).sum() <= 2
    want_dx, want_da, terms = orc.sat_act_backward(g.astype(np.float64), x.astype(np.float64), 15.0, 6.0)
    assert np.array_equal(dx, want_dx.astype(np.float32))
    assert alphas[0] == 6.0
    # two passes of one iteration accumulate: diffAlpha = 2 * sum; the solver ADDS rate/(batch*iterSize)*diff
    assert abs(alphas[1] - 2 * want_da) <= 1e-5 * 2 * np.abs(terms).sum()
    assert abs(alphas[2] - (6.0 + lr / 2 * alphas[1])) <= 1e-6


def test_lsq_quantizer_classes(fh):
    from oracle import oracle as orc
    rng = np.random.default_rng(43)
    w = rng.normal(0, 0.05, size=128 * 64 * 9 + 3).astype(np.float32)
    g = rng.normal(size=w.size).astype(np.float32)
    wq, dw, steps = np.empty_like(w), np.empty_like(w), np.zeros(4, dtype=np.float32)
    assert fh.lib.fh_lsq_cell_run(b"Frame_HIP", w.ctypes.data, g.ctypes.data, w.size, 15, 100.0, 1, wq.ctypes.data, dw.ctypes.data, steps.ctypes.data) == 0
    lo, hi = int(steps[2]), int(steps[3])
    assert (lo, hi) == (-8, 7)
    step0 = 2.0 * np.abs(w.astype(np.float64)).mean() / np.sqrt(hi)          # optimal initial step of the LSQ paper
    assert abs(steps[0] - step0) <= 1e-5 * step0
    want = orc.lsq_forward(w, steps[0], lo, hi)
    assert (np.abs(wq - want) > 1e-5 * np.maximum(np.abs(want), steps[0])).sum() <= 2
    want_dfp, want_sum = orc.lsq_backward(g.astype(np.float64), w.astype(np.float64), float(steps[0]), lo, hi)
    assert np.array_equal(dw, want_dfp.astype(np.float32))
    gs = 1.0 / np.sqrt(w.size * hi)
    assert abs(steps[1] - want_sum * gs) <= 1e-4 * abs(want_sum * gs) + 1e-7
    # activations: range [0, R], fixed step
    x = np.abs(rng.normal(0, 1.0, size=4096)).astype(np.float32)
    gx = rng.normal(size=x.size).astype(np.float32)
    y, dx, st = np.empty_like(x), np.empty_like(x), np.zeros(2, dtype=np.float32)
    assert fh.lib.fh_lsq_act_run(b"Frame_HIP", x.ctypes.data, gx.ctypes.data, x.size, 15, 0.2, 0, y.ctypes.data, dx.ctypes.data, st.ctypes.data) == 0
    assert st[0] == np.float32(0.2)
    want = orc.lsq_forward(x, np.float32(0.2), 0, 15)
    assert (np.abs(y - want) > 1e-5 * np.maximum(np.abs(want), 0.2)).sum() <= 2
    want_dx, want_sum = orc.lsq_backward(gx.astype(np.float64), x.astype(np.float64), float(np.float32(0.2)), 0, 15)
    assert np.array_equal(dx, want_dx.astype(np.float32))
    assert abs(st[1] - want_sum / np.sqrt(x.size * 15)) <= 1e-4 * abs(want_sum / np.sqrt(x.size * 15)) + 1e-7


def test_float_rescaled_net_runs_after_approximation(fh, tmp_path):
    """The ingestion path end to end: integer weights read from N2D2-format text files, FLOAT_MULT rescales (what a
    calibration leaves) turned into 16-bit fixed point by DeepNetQuantization::approximateActivationScaling, the net
    executed on the GPU, and the outputs compared with the CPU oracle running the approximated scalings."""
    from n2d2_amd import nets
    from oracle import cells
    import copy
    spec = copy.deepcopy(nets.lenet())
    net = fh.Net(fh.spec_to_ini(spec, 8))
    rng = np.random.default_rng(51)
    for l in spec.layers:
        if l.type not in ("conv", "fc"):
            if l.type == "pool":
                net.set_quantized(l.name, 8)
            continue
        # parameters through text files, as N2D2 exports them
        np.savetxt(tmp_path / ("%s_weights.syntxt" % l.name), l.w.reshape(l.w.shape[0], -1), fmt="%d")
        np.savetxt(tmp_path / ("%s_biases.syntxt" % l.name), l.bias, fmt="%d")
        net.import_free_parameters(l.name, tmp_path / ("%s.syntxt" % l.name))
        net.set_quantized(l.name, 8, l.act.nb_bits)
        if l.act.mode == "None":
            net.set_scaling(l.name, "None")
            continue
        scale = (np.asarray(l.act.scaling, dtype=np.float64) / 2.0 ** l.act.frac_bits * rng.uniform(0.8, 1.2, size=l.w.shape[0])).astype(np.float32)
        net.set_scaling(l.name, "FloatMult", scale)
        net.approximate_activation_scaling(l.name, "FixedMult16")
        mode, bits, vals = net.scaling(l.name)
        assert mode == "FixedMult16" and abs(vals).max() <= 32767 and abs(vals).max() > 16383
        l.act.mode, l.act.frac_bits, l.act.scaling = mode, bits, vals.astype(np.int64)
    x = rng.integers(0, 256, size=(8, 1, 32, 32))
    net.initialize()
    net.set_stimuli(x)
    net.propagate()
    keep = [l.name for l in spec.layers]
    want = cells.run_net(spec, x, keep=keep)
    # the three FcCells as one launch (the approximated rescales travel with the cells), then every cell on its own
    assert net.nb_folded == 2 and np.array_equal(net.outputs("fc3"), want["fc3"])
    net.set_fusion(False)
    net.propagate()
    for name in keep:
        assert np.array_equal(net.outputs(name), want[name]), name


def test_get_max_output_is_the_first_largest_output(fh):
    from n2d2_amd import nets
    from oracle import cells
    spec = nets.lenet()
    x = np.random.default_rng(41).integers(0, 256, size=(8, 1, 32, 32))
    net = fh.build_net(spec, 8)
    net.initialize()
    net.set_stimuli(x)
    net.propagate()
    last = spec.output
    want = cells.run_net(spec, x, keep=[last, "conv1"])
    for b in range(8):
        assert net.max_output(last, b) == int(np.argmax(want[last][b].reshape(-1)))
        # a saturating feature map has many equal maxima: the first one in (channel, row, column) order counts
        assert net.max_output("conv1", b) == int(np.argmax(want["conv1"][b].reshape(-1)))
    with pytest.raises(fh.FrameHipError):
        net.max_output(last, 8)


def test_replace_input_before_initialize_changes_what_a_cell_reads(fh):
    from n2d2_amd import nets
    from oracle import cells
    b = nets._Builder("rewired", (16, 14, 14), seed=43, scaling_mode="SingleShift")
    b.conv("a", "input", 16, 1)
    b.conv("b", "a", 16, 1)
    b.conv("c", "b", 16, 3, pad=1)
    spec = b.spec
    x = np.random.default_rng(44).integers(0, 256, size=(4, 16, 14, 14))
    net = fh.build_net(spec, 4)
    net.replace_input("c", "b", "a")
    net.initialize()
    net.set_stimuli(x)
    net.propagate()
    straight = cells.run_net(spec, x, keep=["c"])["c"]
    spec.layers[2].inputs = ["a"]
    rewired = cells.run_net(spec, x, keep=["c"])["c"]
    assert not np.array_equal(straight, rewired)
    assert np.array_equal(net.outputs("c"), rewired)
