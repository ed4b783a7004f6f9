"""Model::save_params / save_spec_params / load and the checkpoint directory.

PARITY UNPINNED at the byte level: the reference holds no sample `model.net` / `model.nn` and its writer cannot
run here.  What IS pinned: the section and key order of both files (typed below from the reference's writer,
v1/learner/save.cpp:35-520, independent of the code under test), the CR LF line ends, the 16-digit number format,
the numbering of units and parameters on a hand-checked tiny model, the write -> read -> write round trip
(bit-identical parameters, moving statistics, settings and forward results), the `.tmp` protocol, the refusal of
what this path does not run, and the rotation of the checkpoint directory."""
import os
import re

import numpy as np
import pytest

from oracle.binding import ACT, DROP, NORM, OPT

pytestmark = pytest.mark.gpu

SPEC_SECTIONS = [  # save.cpp:55-165
    ("GRADIENT DESCENT PARAMETERS", ["learning_rate", "learning_rate_final", "learning_momentum", "learning_gamma",
                                     "use_nesterov"]),
    ("QUICKPROP PARAMETERS", ["quickprop_decay", "quickprop_mu"]),
    ("RESILLENT PROPAGATION PARAMETERS", ["rprop_increase_factor", "rprop_decrease_factor", "rprop_delta_min",
                                          "rprop_delta_max", "rprop_delta_zero"]),
    ("SARPROP PARAMETERS", ["sarprop_weight_decay_shift", "sarprop_step_error_threshold_factor",
                            "sarprop_step_error_shift", "sarprop_temperature", "sarprop_epoch"]),
    ("ADAM PARAMETERS", ["adam_learning_rate", "adam_beta1", "adam_beta2", "adam_epsilon", "adam_bias_correction",
                         "adam_gamma"]),
    ("WARM RESTARTS PARAMETERS", ["use_warm_restarts", "warm_restarts_decay_learning_rate",
                                  "warm_restarts_maximum_learning_rate", "warm_restarts_minimum_learning_rate",
                                  "warm_restarts_initial_T_i", "warm_restarts_multiplier"]),
    ("TRAINING PARAMETERS", ["type_optimizer_function", "type_loss_function", "type_accuracy_function",
                             "bit_fail_limit", "pre_training_level", "use_clip_gradient", "clip_gradient"]),
    ("REGULARIZATION PARAMETERS", ["regularization__max_norm_constraints", "regularization__l1", "regularization__l2",
                                   "regularization__srip", "weight_decay", "use_normalized_weight_decay"]),
    ("NORMALIZATION PARAMETERS", ["normalization_momentum_average", "normalization_epsilon",
                                  "batch_renormalization_r_correction_maximum",
                                  "batch_renormalization_d_correction_maximum"]),
    ("LOSS PARAMETERS", ["loss_train", "loss_valid", "loss_testg"]),
    ("ACCURANCY PARAMETERS", ["acc_var", "acc_train", "acc_valid", "acc_testg"]),
    ("COMPUTATION PARAMETERS", ["use_cu", "use_mp", "pct_threads", "maximum_batch_size"]),
]
DIMENSION_KEYS = ["type", "number_layers", "seq_w", "n_time_delay", "use_first_layer_as_input",  # save.cpp:228-244
                  "use_last_layer_as_output", "total_basic_units", "total_basic_indice_units", "total_neuron_units",
                  "total_AF_units", "total_AF_Ind_recurrent_units", "total_block_units", "total_cell_units",
                  "total_normalized_units", "total_parameters", "total_weights", "total_bias"]


@pytest.fixture(scope="module")
def lib(pkg):
    return pkg.load_library()


def read_lines(path):
    raw = open(path, "rb").read()
    assert raw.count(b"\n") == raw.count(b"\r\n"), "every line ends in CR LF"
    return raw.decode("ascii").split("\r\n")


def mlp(lib, widths=(6, 8, 7, 3), train_steps=3):
    from deep_learning_amd.model import Model
    m = Model(lib, list(widths))
    m.set_layer(1, ACT["ELU"], NORM["BRN"], DROP["BERNOULLI"], 0.75)
    m.set_layer(2, ACT["TANH"], NORM["BN"])
    m.set_layer(len(widths) - 1, ACT["SOFTMAX"])
    m.set_norm_hyper(0.9, 1e-4, 3.0, 5.0)
    m.prepare(16)
    m.glorot_uniform(5)
    m.set_optimizer(OPT["ADAM"], adam_lr=0.02, weight_decay=0.01, clip=2.5, max_norm=4.0)
    if train_steps:
        rng = np.random.default_rng(0)
        X = rng.uniform(-1, 1, (48, widths[0])).astype(np.float32)
        Y = np.eye(widths[-1])[rng.integers(0, widths[-1], 48)].astype(np.float32)
        for _ in range(train_steps):
            m.train_epoch(X, Y, resample_masks=True)
    return m


def test_spec_file_has_the_reference_sections_and_keys_in_order(lib, tmp_path):
    m = mlp(lib, train_steps=0)
    try:
        p = tmp_path / "model.nn"
        m.save_spec_params(p)
        lines = read_lines(p)
        expect = []
        for i, (name, keys) in enumerate(SPEC_SECTIONS):
            expect.append("|===| %s |===|" % name)
            expect += keys
            expect.append("|END| %s |END|" % name)
            if i + 1 != len(SPEC_SECTIONS):
                expect.append("")
        expect.append("")  # the text ends with the last line's CR LF
        got = [l if (l.startswith("|") or l == "") else l.split(" ")[0] for l in lines]
        assert got == expect
        fields = dict(l.split(" ") for l in lines if l and not l.startswith("|"))
        # values: what was set above, printed with up to 16 significant digits of the float's exact value
        assert fields["adam_learning_rate"] == "%.16g" % np.float32(0.02)
        assert fields["weight_decay"] == "%.16g" % np.float32(0.01)
        assert fields["clip_gradient"] == "2.5" and fields["use_clip_gradient"] == "1"
        assert fields["regularization__max_norm_constraints"] == "4"
        assert fields["type_optimizer_function"] == str(OPT["ADAM"])
        assert fields["normalization_momentum_average"] == "%.16g" % np.float32(0.9)
        assert fields["batch_renormalization_r_correction_maximum"] == "3"
        assert fields["pct_threads"] == "100" and fields["maximum_batch_size"] == "16"
        assert fields["loss_train"] == "3.40282e+38"  # the reference's start value, FLT_MAX to six digits
    finally:
        m.close()


def test_params_file_of_a_tiny_model_line_by_line(lib, tmp_path):
    """[2 -> 3 (BN, before the activation) -> 2]: every line of the file, with the unit and parameter numbering
    worked out by hand from the reference's layout: weights [3x2 | 2x3], biases [3 | 2], then a scale and a shift
    slot for every unit of every entry (2 + 3 + 2), neuron units numbered through the layers from the inputs."""
    from deep_learning_amd.model import Model
    m = Model(lib, [2, 3, 2])
    try:
        m.set_layer(1, ACT["RELU"], NORM["BN"])
        m.set_layer(2, ACT["LINEAR"])
        m.prepare(4)
        P = np.arange(1, m.P + 1, dtype=np.float32) / 8  # exactly representable, all different
        m.set_parameters(P)
        mean = np.arange(7, dtype=np.float32) + 0.5
        std = np.arange(7, dtype=np.float32) + 2
        m.set_moving(mean, std)
        p = tmp_path / "model.net"
        m.save_params(p)
        lines = read_lines(p)
        assert m.P == 6 + 6 + 3 + 2 + 2 * 7
        g = lambda v: "%.16g" % v
        e = ["|===| DIMENSION |===|", "type 3", "number_layers 3", "seq_w 1", "n_time_delay 0", "use_first_layer_as_input 1",
             "use_last_layer_as_output 1", "total_basic_units 0", "total_basic_indice_units 0", "total_neuron_units 7",
             "total_AF_units 7", "total_AF_Ind_recurrent_units 0", "total_block_units 0", "total_cell_units 0",
             "total_normalized_units 7", "total_parameters 31", "total_weights 12", "total_bias 5",
             "  Input layer:", "    type_layer 3", "    type_activation 0", "    type_dropout 0", "      dropout_values[0] 0",
             "      dropout_values[1] 0", "      dropout_values[2] 0", "    n_inp 2",
             "  Hidden layer 1:", "    type_layer 3", "    use_bidirectional 0", "    type_activation 2", "    type_dropout 0",
             "      use_coded_dropout 0", "      dropout_values[0] 0", "      dropout_values[1] 0", "      dropout_values[2] 0",
             "    type_normalization 1", "      use_layer_normalization_before_activation 1", "      number_normalized_units 3"]
        for k in range(3):  # the hidden layer's units are slots 2..4 of the 7
            e += ["        NormU[%d]" % k, "          scale " + g(P[17 + 2 + k]), "          shift " + g(P[17 + 7 + 2 + k]),
                  "          mean_average[0] " + g(mean[2 + k]), "          variance_average[0] " + g(std[2 + k])]
        e += ["    use_tied_parameter 0", "    k_sparsity 0", "    alpha_sparsity 1", "    constraint_recurrent_weight_lower_bound 0",
              "    constraint_recurrent_weight_upper_bound 0", "    number_neuron_units 3"]
        for j in range(3):
            e += ["      Neuron_unit[%d]" % j, "        number_connections 2"]
            for k in range(2):
                e += ["          connected_to_neuron %d" % k, "          weight[%d] %s" % (2 * j + k, g(P[2 * j + k]))]
        e += ["    number_AF_units 3"]
        for j in range(3):
            e += ["      AF[%d]" % j, "        activation_function %d" % ACT["RELU"]]
        e += ["    number_bias_parameters 3"] + ["      weight[%d] %s" % (12 + j, g(P[12 + j])) for j in range(3)]
        e += ["  Output layer:", "    type_layer 3", "    type_activation 1", "    n_out 2"]
        for j in range(2):
            e += ["      Neuron_unit[%d]" % j, "        number_connections 3"]
            for k in range(3):  # the hidden layer's neuron units are 2..4
                e += ["          connected_to_neuron %d" % (2 + k), "          weight[%d] %s" % (6 + 3 * j + k, g(P[6 + 3 * j + k]))]
        e += ["    number_AF_units 2"]
        for j in range(2):
            e += ["      AF[%d]" % j, "        activation_function %d" % ACT["LINEAR"]]
        e += ["    number_bias_parameters 2"] + ["      weight[%d] %s" % (15 + j, g(P[15 + j])) for j in range(2)]
        e += ["|END| DIMENSION |END|", ""]
        assert lines == e
    finally:
        m.close()


def test_dimension_keys_and_number_format(lib, tmp_path):
    m = mlp(lib)
    try:
        p = tmp_path / "model.net"
        m.save_params(p)
        lines = read_lines(p)
        assert lines[0] == "|===| DIMENSION |===|" and lines[-2] == "|END| DIMENSION |END|"
        assert [l.split(" ")[0] for l in lines[1:1 + len(DIMENSION_KEYS)]] == DIMENSION_KEYS
        # every weight line: the index in brackets addresses the packed parameter array, and the 16 digits
        # bring back the float exactly
        P = m.get_parameters()
        seen = 0
        for l in lines:
            mt = re.fullmatch(r" *weight\[(\d+)\] (\S+)", l)
            if mt:
                assert np.float32(float(mt.group(2))) == P[int(mt.group(1))]
                seen += 1
        assert seen == sum(a * b + b for a, b in zip(m.widths[:-1], m.widths[1:]))
    finally:
        m.close()


def test_round_trip_is_bit_identical(lib, tmp_path):
    from deep_learning_amd.model import Model
    a = mlp(lib)
    b = None
    try:
        a.save_params(tmp_path / "a.net")
        a.save_spec_params(tmp_path / "a.nn")
        b = Model.load(lib, tmp_path / "a.net", tmp_path / "a.nn")
        assert b.widths == a.widths and b.P == a.P and b.n_units == a.n_units
        assert np.array_equal(a.get_parameters(), b.get_parameters())
        for x, y in zip(a.get_moving(), b.get_moving()):
            assert np.array_equal(x, y)
        # writing the loaded model gives the same two files, byte for byte
        b.save_params(tmp_path / "b.net")
        b.save_spec_params(tmp_path / "b.nn")
        for ext in ("net", "nn"):
            assert open(tmp_path / ("a." + ext), "rb").read() == open(tmp_path / ("b." + ext), "rb").read()
        # and the loaded model computes what the saved one computes
        rng = np.random.default_rng(4)
        X = rng.uniform(-1, 1, (16, a.widths[0])).astype(np.float32)
        b.prepare(16)
        a.step(0, X, None, backward=False)  # PROPAGATION::INFERENCE: moving statistics, no dropout
        b.step(0, X, None, backward=False)
        assert np.array_equal(a.get_out(), b.get_out())
    finally:
        a.close()
        if b is not None:
            b.close()


def test_residual_network_round_trip(lib, tmp_path):
    from deep_learning_amd.model import Net
    layers = [("FC", 5), ("FC", 8), ("RES", 2), ("FC", 6), ("FC", 8), ("RES", 2), ("FC", 8), ("FC", 4), ("FC", 3)]
    a = Net(lib, layers)
    b = None
    try:
        for l in a.fc_layers()[:-1]:
            a.set_layer(l, ACT["RELU"], NORM["BN"] if l in (3, 4, 7) else 0)
        a.set_layer(len(layers) - 1, ACT["LINEAR"])
        a.prepare(8)
        a.glorot_uniform(11)
        a.save_params(tmp_path / "r.net")
        a.save_spec_params(tmp_path / "r.nn")
        lines = read_lines(tmp_path / "r.net")
        text = "\n".join(lines)
        # the two RESIDUAL entries carry their depth, the padding of the narrower side and their basic units:
        # entry 2 adds [8] to a block that ends 8 wide; entry 5 adds that [8] to a block that ends 4 wide
        assert "    block_depth 2\n    padding 0\n" in text and "    block_depth 2\n    padding 2\n" in text
        assert text.count("number_basic_units 8") == 2
        fields = dict(l.strip().split(" ") for l in lines[1:18])
        assert fields["total_basic_units"] == "16" and fields["total_neuron_units"] == str(5 + 8 + 6 + 8 + 8 + 4 + 3)
        # activation units: inputs 5, layer 1: 8, first layers of the blocks: none, second ones: their inputs (6, 8),
        # output layer 3
        assert fields["total_AF_units"] == str(5 + 8 + 0 + 6 + 0 + 8 + 3)
        # a layer that reads a block's output is connected to basic units, numbered through the RESIDUAL entries
        assert "connected_to_basic 8" in text and "connected_to_basic 15" in text and "connected_to_basic 16" not in text
        b = Net.load(lib, tmp_path / "r.net", tmp_path / "r.nn")
        assert np.array_equal(a.get_parameters(), b.get_parameters())
        b.save_params(tmp_path / "r2.net")
        assert open(tmp_path / "r.net", "rb").read() == open(tmp_path / "r2.net", "rb").read()
    finally:
        a.close()
        if b is not None:
            b.close()


def edited(src, dst, old, new, count=1):
    raw = open(src, "rb").read()
    assert old.encode() in raw, old
    open(dst, "wb").write(raw.replace(old.encode(), new.encode(), count))


@pytest.mark.parametrize("old,new,which,message", [
    ("    type_layer 3\r\n    use_bidirectional", "    type_layer 7\r\n    use_bidirectional", "net", "FULLY_CONNECTED and LAYER::RESIDUAL"),
    ("k_sparsity 0", "k_sparsity 3", "net", "k-sparse"),
    ("use_tied_parameter 0", "use_tied_parameter 1", "net", "tied"),
    ("use_coded_dropout 0", "use_coded_dropout 1", "net", "coded dropout"),
    ("seq_w 1", "seq_w 4", "net", "seq_w"),
    ("total_parameters ", "total_parameters 1", "net", "total_parameters"),
    ("number_connections 6", "number_connections 5", "net", ""),
    ("connected_to_neuron 1\r\n", "connected_to_neuron 3\r\n", "net", "dense"),
    ("shift ", "shfit ", "net", "can not find `shift`"),
    ("regularization__l1 0", "regularization__l1 0.5", "nn", "L1"),
    ("pre_training_level 0", "pre_training_level 1", "nn", "pre-training"),
    ("adam_beta2", "adam_betta2", "nn", "can not find `adam_beta2`"),
    ("type_optimizer_function 2", "type_optimizer_function 10", "nn", "set_optimizer"),
])
def test_files_this_path_does_not_run_are_refused(lib, tmp_path, old, new, which, message):
    from deep_learning_amd.model import Model
    a = mlp(lib, train_steps=0)
    b = None
    try:
        a.save_params(tmp_path / "a.net")
        a.save_spec_params(tmp_path / "a.nn")
        edited(tmp_path / ("a." + which), tmp_path / ("bad." + which), old, new)
        net = tmp_path / ("bad.net" if which == "net" else "a.net")
        nn = tmp_path / ("bad.nn" if which == "nn" else "a.nn")
        with pytest.raises(RuntimeError) as err:
            b = Model.load(lib, net, nn)
        assert message in str(err.value)
    finally:
        a.close()
        if b is not None:
            b.close()


def test_truncated_file_is_an_error_not_a_crash(lib, tmp_path):
    from deep_learning_amd.model import Model
    a = mlp(lib, train_steps=0)
    try:
        a.save_params(tmp_path / "a.net")
        a.save_spec_params(tmp_path / "a.nn")
        raw = open(tmp_path / "a.net", "rb").read()
        for cut in (len(raw) // 3, len(raw) - 40):
            open(tmp_path / "cut.net", "wb").write(raw[:cut])
            with pytest.raises(RuntimeError):
                Model.load(lib, tmp_path / "cut.net", tmp_path / "a.nn")
        with pytest.raises(RuntimeError):
            Model.load(lib, tmp_path / "missing.net", tmp_path / "a.nn")
    finally:
        a.close()


def test_temp_file_protocol(lib, tmp_path):
    """io/file/file.cpp:63-112, 336-361: while a file is being replaced its old content sits in `<path>.tmp`; a
    finished write removes it; a `.tmp` found by the reader is a write that did not finish, and wins."""
    from deep_learning_amd.model import Model
    a = mlp(lib, train_steps=0)
    b = None
    try:
        net, nn = tmp_path / "m.net", tmp_path / "m.nn"
        a.save_params(net)
        a.save_spec_params(nn)
        good = open(net, "rb").read()
        a.save_params(net)  # replaces an existing file
        assert not os.path.exists(str(net) + ".tmp") and open(net, "rb").read() == good
        # a torn write: the new file is garbage, the previous content is still in .tmp
        open(str(net) + ".tmp", "wb").write(good)
        open(net, "wb").write(good[: len(good) // 2])
        b = Model.load(lib, net, nn)
        assert not os.path.exists(str(net) + ".tmp") and open(net, "rb").read() == good
        assert np.array_equal(a.get_parameters(), b.get_parameters())
    finally:
        a.close()
        if b is not None:
            b.close()


def test_load_into_a_compiled_model_clears_it_first(lib, tmp_path):
    from deep_learning_amd.model import Model
    a = mlp(lib)
    b = Model(lib, [3, 4, 2])
    try:
        b.prepare(4)
        b.glorot_uniform(1)
        a.save_params(tmp_path / "a.net")
        a.save_spec_params(tmp_path / "a.nn")
        assert b.load_files(tmp_path / "a.net", tmp_path / "a.nn")
        assert b.widths == a.widths and np.array_equal(a.get_parameters(), b.get_parameters())
        # and it trains on: one epoch on both from the same state gives the same parameters
        rng = np.random.default_rng(8)
        X = rng.uniform(-1, 1, (32, a.widths[0])).astype(np.float32)
        Y = np.eye(a.widths[-1])[rng.integers(0, a.widths[-1], 32)].astype(np.float32)
        b.prepare(16)
        assert a.evalt(X, Y) == b.evalt(X, Y)
    finally:
        a.close()
        b.close()


def test_checkpoint_directory(lib, tmp_path):
    from deep_learning_amd.model import Checkpointer, Model
    a = mlp(lib, train_steps=0)
    b = Model(lib, [2, 2])
    ck = Checkpointer(a, tmp_path, max_to_keep=5)
    ck2 = Checkpointer(b, tmp_path, max_to_keep=5)
    try:
        assert not ck2.load()  # nothing there yet
        rng = np.random.default_rng(2)
        X = rng.uniform(-1, 1, (32, a.widths[0])).astype(np.float32)
        Y = np.eye(a.widths[-1])[rng.integers(0, a.widths[-1], 32)].astype(np.float32)
        kept = {}
        for step in range(1, 8):
            a.train_epoch(X, Y)
            assert ck.save(step)
            kept[step] = a.get_parameters().copy()
            os.utime(tmp_path / ("ckpt-%d" % step), (1000 + step, 1000 + step))  # distinct write times
        assert sorted(d for d in os.listdir(tmp_path) if d.startswith("ckpt-")) == ["ckpt-%d" % s for s in range(3, 8)]
        assert open(tmp_path / "checkpoint", "rb").read() == b"model_checkpoint_path: ckpt-7"
        assert sorted(os.listdir(tmp_path / "ckpt-7")) == ["model.net", "model.nn"]
        assert ck2.load()
        assert np.array_equal(b.get_parameters(), kept[7])
        # the pointer file decides which one is read
        open(tmp_path / "checkpoint", "wb").write(b"model_checkpoint_path: ckpt-4")
        assert ck2.load()
        assert np.array_equal(b.get_parameters(), kept[4])
    finally:
        ck.close()
        ck2.close()
        a.close()
        b.close()
