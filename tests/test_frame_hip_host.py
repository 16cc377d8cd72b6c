"""The drop-in boundary on the host side, without a GPU: cells are reached through the Registrar under the model key
"Frame_HIP" exactly as N2D2's generators reach "Frame" / "Frame_CUDA"; INI text with DefaultModel=Frame_HIP builds
the net; the signedness decision follows DeepNetExport::isCellOutputUnsigned."""
import pytest


@pytest.fixture(scope="module")
def fh():
    from n2d2_amd import frame_hip
    return frame_hip


INI = """
DefaultModel=%s

[sp]
SizeX=32
SizeY=32
NbChannels=3
BatchSize=2

[conv_def]
Type=Conv
ActivationFunction=Rectifier

[conv1] conv_def
Input=sp
KernelDims=7 7
NbOutputs=16
Stride=2
Padding=3

[pool1]
Input=conv1
Type=Pool
Mapping.ChannelsPerGroup=1
PoolDims=3 3
NbOutputs=16
Stride=2
Pooling=Max

[b_1x1] conv_def
Input=pool1
KernelDims=1 1
NbOutputs=16

[b_x4] conv_def
Input=b_1x1
KernelDims=1 1
NbOutputs=16
ActivationFunction=Linear

[rescale]
Input=pool1
Type=Scaling
NbOutputs=16

[sum]
Input=b_x4,rescale
Type=ElemWise
NbOutputs=16
Operation=Sum
ActivationFunction=Rectifier

[dw] conv_def
Input=sum
KernelDims=3 3
NbOutputs=16
Padding=1
Mapping.ChannelsPerGroup=1

[fc]
Input=dw
Type=Fc
NbOutputs=10
ActivationFunction=Linear
"""


def test_every_class_of_the_path_is_registered_under_frame_hip(fh):
    for t in ("Conv", "Fc", "Pool", "ElemWise", "Scaling", "Rectifier", "Linear", "SATCell", "SATAct", "LSQCell", "LSQAct", "SGDSolver"):
        assert fh.lib.fh_registrar_exists(t.encode(), b"Frame_HIP") == 1, t
        assert fh.lib.fh_registrar_exists(t.encode(), b"Frame_CUDA") == 0, t


def test_the_float_learning_cells_are_registered_under_their_own_key(fh):
    for t in ("Conv", "Fc", "Activation", "Softmax", "BatchNorm", "Pool", "ElemWise"):
        assert fh.lib.fh_train_registrar_exists(t.encode(), b"Frame_HIP_QAT") == 1, t
        assert fh.lib.fh_train_registrar_exists(t.encode(), b"Frame_CUDA") == 0, t
    # the integer inference cells own ("Frame_HIP", float); the two keys do not collide
    assert fh.lib.fh_train_registrar_exists(b"Conv", b"Frame_HIP") == 1
    assert fh.lib.fh_train_registrar_exists(b"Activation", b"Frame_HIP") == 0
    assert fh.lib.fh_train_registrar_exists(b"BatchNorm", b"Frame_HIP") == 0       # the integer graph has none: it is fused away
    assert fh.lib.fh_train_registrar_exists(b"ElemWise", b"Frame_HIP") == 1        # the integer sum cell
    assert fh.lib.fh_train_registrar_exists(b"Scaling", b"Frame_HIP_QAT") == -1    # not a type this query knows


def test_registrar_semantics(fh):
    assert fh.lib.fh_registrar_duplicate_throws() == 1
    assert fh.lib.fh_last_error() == b'Registrar "Frame_HIP" already exists'
    assert fh.lib.fh_registrar_unknown_key_is_null(b"Frame_XYZ") == 1
    assert fh.lib.fh_registrar_unknown_key_is_null(b"Frame_HIP") == 0


def test_ini_default_model_selects_the_cells(fh):
    net = fh.Net(INI % "Frame_HIP")
    assert net.model == "Frame_HIP" and net.nb_cells == 8
    i = net.cell_info("conv1")
    assert (i["W"], i["H"], i["C"], i["B"], i["type"]) == (16, 16, 16, 2, "Conv")
    assert net.cell_info("pool1")["W"] == 7                      # (16 - 3 + 2) / 2, unpadded
    assert net.cell_info("fc")["type"] == "Fc" and net.cell_info("fc")["C"] == 10
    with pytest.raises(fh.FrameHipError) as e:                   # a model nobody registered: the generator's error
        fh.Net(INI % "Frame_CUDA")
    assert 'model "Frame_CUDA" is not valid in section [conv1]' in str(e.value)
    with pytest.raises(fh.FrameHipError):
        fh.Net((INI % "Frame_HIP").replace("Input=pool1\nType=Scaling", "Input=nowhere\nType=Scaling"))
    with pytest.raises(fh.FrameHipError):
        fh.Net((INI % "Frame_HIP").replace("Operation=Sum", "Operation=Prod"))


def test_output_signedness_follows_the_export_globals(fh):
    net = fh.Net(INI % "Frame_HIP")
    import numpy as np
    net.set_scaling("rescale", "FixedMult16", np.full(16, 1 << 13), frac_bits=14)
    try:
        fh.set_globals(8, True, True)
        uns = {n: net.cell_info(n)["unsigned"] for n in ("conv1", "pool1", "b_1x1", "b_x4", "rescale", "sum", "fc")}
        # Rectifier cells unsigned, Linear cells signed, Pool / Scaling inherit from their parents
        assert uns == {"conv1": True, "pool1": True, "b_1x1": True, "b_x4": False, "rescale": True, "sum": True, "fc": False}
        net.set_scaling("rescale", "FixedMult16", -np.full(16, 1 << 13), frac_bits=14)
        assert net.cell_info("rescale")["unsigned"] is False          # a negative factor makes the ScalingCell signed
        fh.set_globals(8, False, True)                                # -no-unsigned: nothing is unsigned
        assert not any(net.cell_info(n)["unsigned"] for n in uns)
        fh.set_globals(0, True, True)                                 # no export precision set: nothing is unsigned
        assert not any(net.cell_info(n)["unsigned"] for n in uns)
    finally:
        fh.set_globals(0, True, False)


# ------------------------------------------------------------------ ingestion of a trained / calibrated network

LENET_INI = """
DefaultModel=Frame_HIP

[sp]
SizeX=32
SizeY=32
NbChannels=1
BatchSize=2

[conv1]
Input=sp
Type=Conv
KernelDims=5 5
NbOutputs=6
NoBias=1
ActivationFunction=Rectifier

[pool1]
Input=conv1
Type=Pool
Mapping.ChannelsPerGroup=1
PoolDims=2 2
NbOutputs=6
Stride=2
Pooling=Max

[conv2]
Input=pool1
Type=Conv
KernelDims=5 5
NbOutputs=16
ActivationFunction=Rectifier

[fc2]
Input=conv2
Type=Fc
NbOutputs=10
NoBias=1
ActivationFunction=Linear
"""


def test_free_parameters_are_read_from_the_reference_s_text_exports(fh, tmp_path):
    """Files exported by N2D2 itself (held by its tests, tests/golden/sat_lenet4b): one line per output, OCHW."""
    import os
    import shutil
    import numpy as np
    golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sat_lenet4b")
    net = fh.Net(LENET_INI)
    # conv1: 6 outputs x 1 channel x 5x5, no bias.  "<dir>/conv1.syntxt" names "<dir>/conv1_weights.syntxt".
    net.import_free_parameters("conv1", os.path.join(golden, "conv1.syntxt"))
    want = np.loadtxt(os.path.join(golden, "conv1_weights.syntxt"), dtype=np.float64).astype(np.float32)
    assert want.shape == (6, 25)
    assert np.array_equal(net.weights("conv1"), want.reshape(-1)) and net.biases("conv1").size == 0
    # conv2 (16 x 6 x 5 x 5) has a bias here and the export holds none: the reference's error for the missing file
    shutil.copy(os.path.join(golden, "conv2_weights.syntxt"), tmp_path / "conv2_weights.syntxt")
    with pytest.raises(fh.FrameHipError) as e:
        net.import_free_parameters("conv2", tmp_path / "conv2.syntxt")
    assert str(e.value) == "Could not open synaptic file: %s" % (tmp_path / "conv2_biases.syntxt")
    np.savetxt(tmp_path / "conv2_biases.syntxt", np.arange(16) * 0.5 - 3)
    net.import_free_parameters("conv2", tmp_path / "conv2.syntxt")
    want2 = np.loadtxt(os.path.join(golden, "conv2_weights.syntxt")).astype(np.float32)
    assert want2.shape == (16, 150)
    assert np.array_equal(net.weights("conv2"), want2.reshape(-1))
    assert np.array_equal(net.biases("conv2"), (np.arange(16) * 0.5 - 3).astype(np.float32))
    # one file holding weights then the bias of each output is read too (singleFile)
    rows = [" ".join("%r" % float(v) for v in want2[o]) + " %r" % (o + 0.25) for o in range(16)]
    (tmp_path / "both.syntxt").write_text("\n".join(rows) + "\n")
    net.import_free_parameters("conv2", tmp_path / "both.syntxt")
    assert np.array_equal(net.weights("conv2"), want2.reshape(-1)) and np.array_equal(net.biases("conv2"), np.arange(16, dtype=np.float32) + 0.25)
    # the reference's other errors
    with pytest.raises(fh.FrameHipError) as e:
        net.import_free_parameters("conv1", tmp_path / "nothing.syntxt")
    assert str(e.value) == "Could not open synaptic file: %s" % (tmp_path / "nothing_weights.syntxt")
    net.import_free_parameters("conv1", tmp_path / "nothing.syntxt", ignore_not_exists=True)      # a notice, no error
    (tmp_path / "short_weights.syntxt").write_text("1 2 3\n")
    with pytest.raises(fh.FrameHipError) as e:
        net.import_free_parameters("conv1", tmp_path / "short.syntxt")
    assert "Error while reading synaptic file" in str(e.value)
    (tmp_path / "long_weights.syntxt").write_text(" ".join(["1"] * 151) + "\n")
    with pytest.raises(fh.FrameHipError) as e:
        net.import_free_parameters("conv1", tmp_path / "long.syntxt")
    assert "Synaptic file size larger than expected" in str(e.value)
    assert np.array_equal(net.weights("conv1"), want.reshape(-1))                                  # a failed import changes nothing
    # fc2: 10 outputs x 84 inputs would need an 84-input cell; here the cell has 16*10*10 inputs, so the file is short
    with pytest.raises(fh.FrameHipError):
        net.import_free_parameters("fc2", os.path.join(golden, "fc2.syntxt"))
    # export -> import round trip, 10 significant digits as the reference writes quantized cells
    net.export_free_parameters("conv2", tmp_path / "rt.syntxt")
    before_w, before_b = net.weights("conv2"), net.biases("conv2")
    net.import_free_parameters("conv2", tmp_path / "conv2.syntxt")
    net.import_free_parameters("conv2", tmp_path / "rt.syntxt")
    assert np.allclose(net.weights("conv2"), before_w, rtol=1e-9, atol=0) and np.array_equal(net.biases("conv2"), before_b)


def test_float_rescales_become_integer_scalings_as_in_the_reference(fh):
    """DeepNetQuantization::approximateActivationScaling: the Scaling that replaces a FLOAT_MULT one, and the per-output
    correction of the cell's parameters for the shift modes, against the oracle's restatement."""
    import numpy as np
    from oracle import ptq_scaling as ref
    rng = np.random.default_rng(17)
    for mode in ("FixedMult16", "FixedMult32", "SingleShift", "DoubleShift", "FloatMult"):
        net = fh.Net(LENET_INI)
        w = rng.normal(0, 20, size=(16, 6, 5, 5)).astype(np.float32)
        b = rng.normal(0, 100, size=16).astype(np.float32)
        net.set_weights("conv2", w)
        net.set_biases("conv2", b)
        sc = np.exp(rng.uniform(-7, 0, size=16)).astype(np.float32)
        net.set_scaling("conv2", "FloatMult", sc)
        net.approximate_activation_scaling("conv2", mode)
        want_mode, want_vals, want_bits, rescale = ref.approximate_activation_scaling(sc, mode)
        got_mode, got_bits, got_vals = net.scaling("conv2")
        assert got_mode == want_mode and got_bits == want_bits
        assert np.array_equal(got_vals.reshape(np.asarray(want_vals).shape), np.asarray(want_vals, dtype=np.float64)), mode
        assert np.array_equal(net.weights("conv2").reshape(16, -1), w.reshape(16, -1) * rescale[:, None]), mode
        assert np.array_equal(net.biases("conv2"), b * rescale), mode
        if mode == "DoubleShift":
            # the pair is (difference, larger exponent): x * (2^-e0 + 2^-e1) = (x + (x << (e1 - e0))) >> e1
            assert (got_vals.reshape(16, 2)[:, 0] <= got_vals.reshape(16, 2)[:, 1]).all()
    # a factor above 1 cannot be a shift: the cell falls back to 16-bit fixed point, parameters untouched
    net = fh.Net(LENET_INI)
    w = rng.normal(0, 20, size=(16, 6, 5, 5)).astype(np.float32)
    net.set_weights("conv2", w)
    net.set_scaling("conv2", "FloatMult", np.linspace(0.5, 1.5, 16).astype(np.float32))
    net.approximate_activation_scaling("conv2", "SingleShift")
    mode, bits, vals = net.scaling("conv2")
    assert mode == "FixedMult16" and bits == 14 and vals[-1] == 1.5 * 2 ** 14 and np.array_equal(net.weights("conv2"), w.reshape(-1))
    # an activation without a floating-point scaling is refused
    with pytest.raises(fh.FrameHipError):
        net.approximate_activation_scaling("conv2", "SingleShift")


def test_the_inference_cells_refuse_a_learning_pass(fh):
    net = fh.Net(INI % "Frame_HIP")
    for call in (net.back_propagate, net.update, net.check_gradient):
        with pytest.raises(fh.FrameHipError) as e:
            call("conv1")
        assert "conv1" in str(e.value) and "quantized inference" in str(e.value)
    with pytest.raises(fh.FrameHipError) as e:
        net.back_propagate("sum")
    assert "Frame_HIP_QAT" in str(e.value)


def test_replace_input_rewires_a_cell_as_cell_frame_does(fh):
    net = fh.Net(INI % "Frame_HIP")
    before = net.cell_info("b_x4")
    net.replace_input("b_x4", "b_1x1", "pool1")            # same 16 x 7 x 7 tensor from another producer
    assert net.cell_info("b_x4") == before
    with pytest.raises(fh.FrameHipError) as e:              # b_x4 no longer reads b_1x1: the reference's message
        net.replace_input("b_x4", "b_1x1", "pool1")
    assert "can't replace input, the input has not been found." in str(e.value)
    with pytest.raises(fh.FrameHipError) as e:              # one input of a sum may not change the output's size
        net.replace_input("sum", "rescale", "conv1")
    assert "the output dimension has changed and doesn't match the other inputs!" in str(e.value)
    assert net.cell_info("sum")["W"] == 7                   # and the failed call leaves the cell as it was
    net.replace_input("dw", "sum", "conv1")                 # a single-input cell follows its new input's size
    assert (net.cell_info("dw")["W"], net.cell_info("dw")["H"]) == (16, 16)


def test_get_nb_groups_from_a_connection_map_against_the_oracle(fh):
    """Cell::getNbGroups (src/Cell/Cell.cpp:251-300) in the cell layer: equal diagonal blocks give their count, an
    unconnected first output gives 0, and every other map is counted by hand (getNbGroupsHandMade, `:178-249`), as the
    oracle's restatements of the two functions say; a map on which the reference's hand count does not return is refused by
    both."""
    import numpy as np
    from oracle import oracle as orc
    rng = np.random.default_rng(5)

    def block_map(O, Cn, G):
        m = np.zeros((O, Cn), dtype=np.uint8)
        for g in range(G):
            m[g * (O // G):(g + 1) * (O // G), g * (Cn // G):(g + 1) * (Cn // G)] = 1
        return m

    def same_as_oracle(m):          # m: [outputs, channels]; the oracle takes [channels, outputs]
        want = orc.get_nb_groups(m.T)
        if want >= 0:
            assert fh.get_nb_groups(m, with_regular=True) == (want, True)
            return
        try:
            by_hand = orc.get_nb_groups_hand_made(m.T)
        except ValueError:
            with pytest.raises(fh.FrameHipError, match="does not return"):
                fh.get_nb_groups(m)
            return
        assert fh.get_nb_groups(m, with_regular=True) == (by_hand, False)

    for (O, Cn, G) in ((8, 8, 8), (12, 6, 3), (6, 12, 2), (5, 7, 1), (64, 64, 64), (16, 4, 4), (4, 16, 4)):
        m = block_map(O, Cn, G)
        assert fh.get_nb_groups(m) == G == orc.get_nb_groups(m.T)
        # any single flipped connection makes it irregular (or moves the first run, which must break a later row)
        for _ in range(6):
            o, c = int(rng.integers(0, O)), int(rng.integers(0, Cn))
            bad = m.copy()
            bad[o, c] ^= 1
            same_as_oracle(bad)
    for _ in range(300):
        O, Cn = int(rng.integers(1, 9)), int(rng.integers(1, 9))
        same_as_oracle((rng.random((O, Cn)) < rng.uniform(0.2, 0.8)).astype(np.uint8))
    assert fh.get_nb_groups(np.zeros((4, 6), dtype=np.uint8)) == 0
    # unequal blocks: the regular test fails, the hand count says 2
    uneven = np.zeros((4, 4), dtype=np.uint8)
    uneven[0:1, 0:1] = 1
    uneven[1:4, 1:4] = 1
    assert orc.get_nb_groups(uneven.T) == -1 and fh.get_nb_groups(uneven, with_regular=True) == (2, False)


def test_conv_mapping_sets_the_groups(fh):
    import numpy as np
    net = fh.Net((INI % "Frame_HIP"))
    info = net.cell_info("conv1")
    O, Cn = 16, 3
    net.set_mapping("conv1", np.tri(O, Cn))             # not a set of equal groups: kept, the cell skips the missing connections
    hole = np.tri(O, Cn)
    hole[5, :] = 0
    with pytest.raises(fh.FrameHipError, match="does not return"):      # (the reference's hand count spins on such a map)
        net.set_mapping("conv1", hole)
    with pytest.raises(fh.FrameHipError, match="is not connected"):
        net.set_mapping("conv1", np.tri(O, Cn)[::-1].copy() * 0 + np.eye(O, Cn, k=-1))
    with pytest.raises(fh.FrameHipError, match="must be"):
        net.set_mapping("conv1", np.ones((O + 1, Cn)))
    net.set_mapping("conv1", np.ones((O, Cn)))          # fully connected: one group
    net.set_mapping("pool1", np.ones((16, 16)))         # a PoolCell takes a map too: every channel behind every output
    with pytest.raises(fh.FrameHipError, match="must be"):
        net.set_mapping("pool1", np.ones((16, 15)))
    with pytest.raises(fh.FrameHipError, match="neither a Conv nor a Pool"):
        net.set_mapping("fc", np.ones((16, 16)))


def test_grouped_conv_sections_are_checked_as_the_generator_does(fh):
    """Conv sections with Mapping.NbGroups / Mapping.ChannelsPerGroup: channels the groups do not divide are refused
    (src/Generator/MappingGenerator.cpp:110-128 throws there; an integer division would quietly make other groups), and so
    is a grouped Conv over several parents, whose groups the reference lays per parent."""
    ini = INI % "Frame_HIP"
    ok = ini.replace("[dw] conv_def\nInput=sum\nKernelDims=3 3\nNbOutputs=16\nPadding=1\nMapping.ChannelsPerGroup=1",
                     "[dw] conv_def\nInput=sum\nKernelDims=3 3\nNbOutputs=16\nPadding=1\nMapping.ChannelsPerGroup=4")
    assert ok != ini
    fh.Net(ok)                                          # 16 channels in groups of 4: accepted
    with pytest.raises(fh.FrameHipError, match="must be a multiple of the number of input channels"):
        fh.Net(ok.replace("Mapping.ChannelsPerGroup=4", "Mapping.ChannelsPerGroup=5"))
    with pytest.raises(fh.FrameHipError, match="must be a multiple of the number of input channels"):
        fh.Net(ok.replace("Mapping.ChannelsPerGroup=4", "Mapping.NbGroups=3"))
    with pytest.raises(fh.FrameHipError, match="several parents"):
        fh.Net(ok.replace("[dw] conv_def\nInput=sum", "[dw] conv_def\nInput=sum,pool1"))


def test_quantization_files_round_trip(fh, tmp_path):
    """DeepNet::saveQuantization / loadQuantization: what the quantization pass leaves in the cells beside their weights
    (bit widths, Scaling mode, factors, fractional bits, clip) goes through one text file per cell and comes back bit
    for bit, for every scaling mode; damaged files are refused with a message naming the file."""
    import numpy as np
    rng = np.random.default_rng(3)
    net = fh.Net(INI % "Frame_HIP")
    cells = {"conv1": 16}
    info = net.cell_info("conv1")
    settings = [("FloatMult", rng.uniform(1e-4, 0.3, 16).astype(np.float32), 0, rng.uniform(1.0, 300.0, 16).astype(np.float32)),
                ("FixedMult16", rng.integers(1, 2 ** 15, 16).astype(np.int32), 13, None),
                ("FixedMult32", rng.integers(-2 ** 20, 2 ** 30, 16).astype(np.int32), 27, rng.uniform(1.0, 300.0, 16).astype(np.float32)),
                ("SingleShift", rng.integers(0, 20, 16).astype(np.uint8), 0, None),
                ("DoubleShift", rng.integers(0, 12, (16, 2)).astype(np.uint8), 0, None),
                ("None", None, 0, None)]
    for k, (mode, scaling, frac, clip) in enumerate(settings):
        net.set_scaling("conv1", mode, scaling, frac, clip)
        net.set_quantized("conv1", 8, 4 + k % 5)
        d = tmp_path / ("q%d" % k)
        d.mkdir()
        net.save_quantization(d)
        assert (d / "conv1.quant").exists() and (d / "pool1.quant").exists()
        other = fh.Net(INI % "Frame_HIP")
        other.load_quantization(d)
        m2, f2, v2 = other.scaling("conv1")
        assert m2 == mode
        if mode != "None":
            assert f2 == (frac if mode.startswith("Fixed") else 0)
            assert np.array_equal(v2.astype(np.float32), np.asarray(scaling).reshape(-1).astype(np.float32))
            c2 = other.clipping("conv1")
            assert (c2 is None) == (clip is None) and (clip is None or np.array_equal(c2, clip))
        assert other.quantized("conv1")[:2] == (8, 4 + k % 5)
    # a file that announces more values than it holds, a missing file, a scaling for another cell size
    d = tmp_path / "bad"
    d.mkdir()
    net.set_scaling("conv1", "SingleShift", np.arange(16, dtype=np.uint8))
    net.save_quantization(d)
    text = (d / "conv1.quant").read_text()
    (d / "conv1.quant").write_text(text.replace("Scaling=16", "Scaling=17"))
    with pytest.raises(fh.FrameHipError, match="announces 17 values and holds 16"):
        fh.Net(INI % "Frame_HIP").load_quantization(d)
    (d / "conv1.quant").write_text(text.replace("Scaling=16 0", "Scaling=15"))
    with pytest.raises(fh.FrameHipError, match="holds a scaling for 15 outputs"):
        fh.Net(INI % "Frame_HIP").load_quantization(d)
    (d / "conv1.quant").write_text(text.replace("IsClipped=0\n", ""))
    with pytest.raises(fh.FrameHipError, match="Missing key IsClipped"):
        fh.Net(INI % "Frame_HIP").load_quantization(d)
    (d / "conv1.quant").unlink()
    with pytest.raises(fh.FrameHipError, match="Could not open quantization file"):
        fh.Net(INI % "Frame_HIP").load_quantization(d)
