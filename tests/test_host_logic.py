"""CPU-only checks of the Python host layer (the mirror of the reference's deepshift package)."""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn as nn

import deepshift_amd
from deepshift_amd import convert, kernels, modules, modules_q, utils, workloads

HERE = os.path.dirname(os.path.abspath(__file__))
KAT = json.load(open(os.path.join(HERE, "golden", "kat.json")))


@pytest.mark.parametrize("case", KAT["round_to_fixed"], ids=lambda c: "I%dF%d" % (c["I"], c["F"]))
def test_round_to_fixed_known_answers(case):
    got = utils.round_to_fixed(torch.tensor(case["x"], dtype=torch.float32), case["I"], case["F"])
    np.testing.assert_array_equal(got.numpy(), np.array(case["y"], np.float32))


def test_round_to_fixed_matches_oracle(oracle, rng):
    x = (rng.standard_normal(5000) * rng.choice([1e-4, 1.0, 1e3, 1e6], size=5000)).astype(np.float32)
    for I, F in [(16, 16), (3, 5), (8, 8), (1, 4)]:
        np.testing.assert_array_equal(utils.round_to_fixed(torch.from_numpy(x), I, F).numpy(),
                                      oracle.round_to_fixed(x, I, F))


def test_get_shift_and_sign_known_answers():
    k = KAT["shift_and_sign"]
    shift, sign = utils.get_shift_and_sign(torch.tensor(k["w"], dtype=torch.float32))
    np.testing.assert_array_equal(shift.numpy(), np.array(k["shift"], np.float32))
    np.testing.assert_array_equal(sign.numpy(), np.array(k["sign"], np.float32))
    shift, sign = utils.get_shift_and_sign(torch.zeros(1))
    assert shift.item() == -np.inf and sign.item() == 0
    np.testing.assert_array_equal(utils.round_power_of_2(torch.tensor([0.7, -0.1, 3.0])).numpy(),
                                  np.array([0.5, -0.125, 4.0], np.float32))


def test_bits_table():
    for k, v in KAT["bits_from_min_shift"]["table"].items():
        assert utils.shift_field_bits(int(k)) == v, k


def test_clampabs_and_round():
    x = torch.tensor([-3.0, -0.001, 0.0, 0.002, 0.5, 7.0])
    np.testing.assert_allclose(utils.clampabs(x.clone(), 0.01, 1.0).numpy(), [-1, -0.01, 0, 0.01, 0.5, 1])
    np.testing.assert_array_equal(utils.round(torch.tensor([0.5, 1.5, 2.5, -0.5])).numpy(), [0, 2, 2, -0])
    r = utils.round(torch.full((1000,), 0.25), 'stochastic')
    assert set(r.unique().tolist()) <= {0.0, 1.0} and 100 < r.sum() < 400


def test_module_constructors_mirror_reference_defaults():
    lin = modules.LinearShift(7, 5)
    assert lin.shift.shape == (5, 7) and lin.sign.shape == (5, 7) and lin.bias.shape == (5,)
    assert lin.shift_range == (-14, 0) and lin.conc_weight is None and lin.use_kernel is False
    assert modules.LinearShift(7, 5, weight_bits=3).shift_range == (-2, 0)
    assert modules_q.LinearShiftQ(7, 5, weight_bits=3).shift_range == (-3, 0)
    conv = modules.Conv2dShift(3, 8, 3, stride=2, padding=1, bias=False)
    assert conv.shift.shape == (8, 3, 3, 3) and conv.bias is None and conv.stride == (2, 2)
    assert "kernel_size=(3, 3)" in repr(conv)
    assert not modules.LinearShift(3, 2, freeze_sign=True).sign.requires_grad
    assert modules.LinearShift(3, 2, check_grad=True).shift.dtype == torch.float64
    with pytest.raises(ValueError):
        modules.Conv2dShift(3, 8, 3, groups=2)


def test_float_paths_use_power_of_two_weights():
    torch.manual_seed(0)
    lin = modules.LinearShift(6, 4)
    x = torch.randn(3, 6)
    w = 2.0 ** lin.shift.data.clamp(-14, 0).round() * lin.sign.data.round().sign()
    torch.testing.assert_close(lin(x), x @ w.t() + lin.bias)
    conv = modules.Conv2dShift(2, 3, 3, padding=1)
    xi = torch.randn(1, 2, 5, 5)
    w = 2.0 ** conv.shift.data.round() * conv.sign.data.round().sign()
    want = torch.nn.functional.conv2d(utils.round_to_fixed(xi), w, utils.round_to_fixed(conv.bias.data), padding=1)
    torch.testing.assert_close(conv(xi), want)
    q = modules_q.Conv2dShiftQ(2, 3, 3, padding=1)
    wq = utils.round_power_of_2(utils.clampabs(q.weight.data.clone(), 2.0 ** -15, 1.0))
    want = torch.nn.functional.conv2d(utils.round_to_fixed(xi), wq, utils.round_to_fixed(q.bias.data), padding=1)
    torch.testing.assert_close(q(xi), want)
    # gradients flow straight through the rounding
    lin(x).sum().backward()
    assert lin.shift.grad is not None and lin.sign.grad is not None


def test_convert_to_shift_walks_backwards_and_counts():
    model = nn.Sequential(nn.Conv2d(3, 4, 3), nn.ReLU(), nn.Conv2d(4, 4, 3), nn.Flatten(), nn.Linear(16, 2))
    m, n = convert.convert_to_shift(model, shift_depth=1, shift_type='PS', convert_weights=True)
    # the LAST conv is converted first; linears are always converted with convert_all_linear
    assert n == 1
    assert type(m[0]) is nn.Conv2d and type(m[2]) is modules.Conv2dShift and type(m[4]) is modules.LinearShift
    assert convert.count_layer_type(m, modules.Conv2dShift) == 1
    model = workloads.ResNet20()
    w0 = model.stem[0].weight.detach().clone()
    m, n = convert.convert_to_shift(model, 1000, 'PS', convert_weights=True)
    assert n == 19 and convert.count_layer_type(m, modules.Conv2dShift) == 19
    assert convert.count_layer_type(m, modules.LinearShift) == 1
    shift, sign = utils.get_shift_and_sign(w0)
    torch.testing.assert_close(m.stem[0].shift.data, shift)
    torch.testing.assert_close(m.stem[0].sign.data, sign)
    mq, n = convert.convert_to_shift(workloads.MLP(), 0, 'Q')
    assert n == 0 and convert.count_layer_type(mq, modules_q.LinearShiftQ) == 3
    with pytest.raises(ValueError):
        convert.convert_to_shift(nn.Sequential(nn.Linear(2, 2)), 1, 'XYZ')


def test_round_shift_weights():
    torch.manual_seed(1)
    model = nn.Sequential(modules.Conv2dShift(2, 2, 3), modules_q.LinearShiftQ(4, 3))
    model[0].shift.data += 0.3
    out = convert.round_shift_weights(model, clone=True)
    assert torch.equal(out[0].shift.data, out[0].shift.data.round())
    assert set(out[0].sign.data.unique().tolist()) <= {-1.0, 0.0, 1.0}
    w = out[1].weight.data
    assert torch.equal(w.abs().log2(), w.abs().log2().round())
    assert torch.equal(out[0].bias.data, utils.round_to_fixed(out[0].bias.data))
    assert not torch.equal(model[0].shift.data, out[0].shift.data)  # clone left the original alone


def test_gpu_kernel_path_never_falls_back_to_the_host():
    """use_cuda=True with CPU tensors is an error, not a silent host computation (use_cuda=False is
    the explicit way to the host kernels, tests/test_cpu_twin.py)."""
    with pytest.raises((ValueError, RuntimeError, AssertionError)):
        kernels.linear(torch.zeros(1, 1, dtype=torch.int32), torch.zeros(1, 1), torch.zeros(1, 1),
                       conc_weight=utils.ConcWeight(torch.zeros(1, dtype=torch.int32), 0, 4))
    lin = modules.LinearShift(4, 3, use_kernel=True, use_cuda=True)
    with pytest.raises((ValueError, RuntimeError, TypeError, AssertionError)):
        lin(torch.randn(2, 4))


def test_packed_weights_follow_the_parameters():
    """conc_weight assigned from outside is kept; one built from the layer's parameters carries the
    key of those parameters so that a later change repacks."""
    lin = modules.LinearShift(4, 3, use_kernel=True)
    assert lin.conc_weight is None and lin._packed_from is None
    given = utils.ConcWeight(torch.zeros(3, dtype=torch.int32), 0, 4)
    lin.conc_weight = given
    assert lin.packed_weights() is given       # nothing to compare against: used as given
    key = modules._params_key(lin.shift, lin.sign)
    with torch.no_grad():
        lin.shift.add_(1.0)                    # what an optimizer step or load_state_dict does
    assert modules._params_key(lin.shift, lin.sign) != key
    lin.load_state_dict(lin.state_dict())
    assert "conc_weight" not in lin.state_dict() and "_conc_weight" not in lin.state_dict()


def test_workload_pair_counts():
    for cls, chw, batch, want in [(workloads.ResNet18, (3, 224, 224), 64, 116.1e9),
                                  (workloads.ResNet20, (3, 32, 32), 256, 10.38e9),
                                  (workloads.MLP, (784,), 64, 42.8e6)]:
        shapes = workloads.shift_layer_shapes(cls(), chw, batch)
        pairs = sum(l["M"] * l["K"] * l["N"] for l in shapes)
        assert abs(pairs - want) / want < 2e-3
    assert deepshift_amd.__version__


def test_fused_graph_hands_fixed_point_tensors_on():
    """Structure of the fused ResNet-18 graph (no kernel runs): every block's first convolution
    takes its producer's int32 tensor, and the float result is kept only where a shortcut needs it."""
    from deepshift_amd import convert, fuse, modules, workloads
    model = workloads.ResNet18()
    model, n = convert.convert_to_shift(model, 1000, 'PS', convert_weights=False, use_kernel=False)
    for m in model.modules():
        if isinstance(m, (modules.Conv2dShift, modules.LinearShift)):
            m.use_kernel = True
    gm = fuse.fuse_conv_epilogues(model)
    fused = [m for m in gm.modules() if isinstance(m, fuse.FusedConv2dShift)]
    assert len(fused) == 20
    assert sum(m.prequantized for m in fused) == 16          # 8 second convolutions + 8 block inputs
    emits = [m.emit for m in fused if m.emit is not None]
    assert len(emits) == 16 and sum(e[3] for e in emits) == 8  # float kept for the 8 block inputs
    assert [m.pool for m in fused if m.pool] == [(3, 2, 1)]    # the stem's max pooling rides along
    assert all(e[:3] == ((1, 1), 16, 16) for e in emits)
    plain = fuse.fuse_conv_epilogues(model, handoff=False)
    assert not any(m.prequantized or m.emit for m in plain.modules() if isinstance(m, fuse.FusedConv2dShift))


def test_evaluate_cli_arguments_and_refusals():
    from deepshift_amd import evaluate
    args = evaluate.build_parser().parse_args(["-e", "-a", "resnet20", "--use-kernel", "True", "-wb", "3",
                                               "-ab", "3", "5", "--shift-depth", "0"])
    assert args.evaluate and args.use_kernel is True and args.activation_bits == [3, 5]
    assert args.arch == "resnet20" and args.shift_depth == 0 and args.weight_bits == 3
    with pytest.raises(SystemExit) as e:
        evaluate.main([])
    assert "evaluate" in str(e.value)
    if not torch.cuda.is_available():
        with pytest.raises(SystemExit) as e:
            evaluate.main(["-e"])
        assert "GPU" in str(e.value)


def test_packed_export_rejects_foreign_files(tmp_path):
    from deepshift_amd import export, workloads
    torch.save({"format": "something else", "layers": {}}, tmp_path / "x.pt")
    with pytest.raises(ValueError):
        export.load_packed(workloads.MLP(), str(tmp_path / "x.pt"))
    torch.save({"format": export.FORMAT, "layers": {"nope": {}}}, tmp_path / "y.pt")
    with pytest.raises(KeyError):
        export.load_packed(workloads.MLP(), str(tmp_path / "y.pt"))


def test_int8_kernel_eligibility():
    """kernels.paired_fields: activations of at most 8 bits (not the one-bit format), a multiple of 64
    channels, base 0, shift fields of at most 4 bits (packed that narrow, or ternary 6-bit words whose
    non-zero fields are), the highest value of a 3- or 4-bit field unused."""
    from deepshift_amd import kernels
    from deepshift_amd.utils import ConcWeight
    narrow = ConcWeight(None, 0, 2)
    assert kernels.paired_fields(narrow, 64, 3, 5) == (2, 2)
    assert kernels.paired_fields(ConcWeight(None, 0, 1), 128, 2, 6) == (1, 1)
    assert kernels.paired_fields(narrow, 64, 16, 16) is None      # 32-bit activations
    assert kernels.paired_fields(narrow, 64, 1, 7) is None        # sign(x) - 1 reaches -2 * 2^F
    assert kernels.paired_fields(narrow, 64, 4, 5) is None        # 9 bits
    assert kernels.paired_fields(narrow, 96, 3, 5) is None        # channels
    assert kernels.paired_fields(ConcWeight(None, -1, 2), 64, 3, 5) is None
    assert kernels.paired_fields(ConcWeight(None, 0, 3), 64, 3, 5) is None            # top field unknown
    assert kernels.paired_fields(ConcWeight(None, 0, 3, max_field=7), 64, 3, 5) is None
    assert kernels.paired_fields(ConcWeight(None, 0, 3, max_field=6), 64, 3, 5) == (3, 3)
    assert kernels.paired_fields(ConcWeight(None, 0, 4, max_field=14), 64, 3, 5) == (4, 4)
    assert kernels.paired_fields(ConcWeight(None, 0, 4, max_field=15), 64, 3, 5) is None
    assert kernels.paired_fields(ConcWeight(None, 0, 5, max_field=20), 64, 3, 5) is None
    assert kernels.paired_fields(None, 64, 3, 5) is None
    assert kernels.paired_fields(ConcWeight(None, 0, 6, 2), 64, 3, 5) == (6, 2 | 0x200)  # fields <= 2: 3 is free
    assert kernels.paired_fields(ConcWeight(None, 0, 2, max_field=2), 64, 3, 5) == (2, 2 | 0x200)
    assert kernels.paired_fields(ConcWeight(None, 0, 2, max_field=3), 64, 3, 5) == (2, 2)
    assert kernels.paired_fields(ConcWeight(None, 0, 1, max_field=0), 64, 3, 5) == (1, 1 | 0x200)
    assert kernels.paired_fields(ConcWeight(None, 0, 6, 4), 64, 3, 5) == (6, 4)
    assert kernels.paired_fields(ConcWeight(None, 0, 6, 0), 64, 3, 5) is None


def test_small_layers_stay_on_the_int32_kernels():
    """modules._small_for_int8: few 384-pixel x 64-channel tiles and a short reduction."""
    from deepshift_amd import modules
    shortcut = modules.Conv2dShift(64, 128, 1, stride=2, use_kernel=True)
    assert modules._small_for_int8(shortcut, (64, 64, 56, 56), 4)          # ResNet-18 1x1/2 shortcut
    body = modules.Conv2dShift(512, 512, 3, padding=1, use_kernel=True)
    assert not modules._small_for_int8(body, (64, 512, 7, 7), 4)           # few tiles, K = 4608
    assert modules._small_for_int8(body, (1, 512, 7, 7), 4)                # batch 1
    wide = modules.Conv2dShift(64, 256, 1, use_kernel=True)
    assert not modules._small_for_int8(wide, (128, 64, 56, 56), 2)         # ResNet-50 stage 1


def test_small_linear_routing_respects_the_one_launch_kernels_limits():
    """linear_layer sends a layer to ds_linear_small_f32 only below the break-even in pairs AND within that
    entry point's limits (65535 workgroup rows of 64 batch rows, 32-bit byte offsets); a tiny layer applied
    to millions of rows stays on the tiled path, which served it before."""
    assert kernels.small_linear_serves(64, 784, 512)
    assert kernels.small_linear_serves(128, 2048, 1000)
    assert not kernels.small_linear_serves(1024, 1024, 1024)            # above the break-even
    assert kernels.small_linear_serves(65535 * 64, 8, 8)
    assert not kernels.small_linear_serves(65535 * 64 + 1, 8, 8)        # gridDim.y
    assert not kernels.small_linear_serves(5_000_000, 8, 8)
    assert not kernels.small_linear_serves(2 ** 20, 512, 1)             # M * K * 4 = 2^31
    assert not kernels.small_linear_serves(2 ** 20, 1, 512)             # M * N * 4 = 2^31


def test_kept_hand_off_buffer_is_not_reused_while_its_last_result_is_alive():
    cache = {}
    a = kernels._kept_padded_buffer(cache, (1, 2, 4, 4), torch.int32, torch.device("cpu"))
    assert a.shape == (1, 2, 4, 4) and not a.any()
    ptr_a = a.data_ptr()
    del a
    b = kernels._kept_padded_buffer(cache, (1, 2, 4, 4), torch.int32, torch.device("cpu"))
    assert b.data_ptr() == ptr_a, "nobody held the buffer: reused"
    b.fill_(7)
    c = kernels._kept_padded_buffer(cache, (1, 2, 4, 4), torch.int32, torch.device("cpu"))
    assert c.data_ptr() != b.data_ptr() and not c.any(), "the earlier result is alive: a fresh zeroed buffer"
    assert bool((b == 7).all())
    view = c[:, :1]
    del c
    d = kernels._kept_padded_buffer(cache, (1, 2, 4, 4), torch.int32, torch.device("cpu"))
    assert d.data_ptr() != view.data_ptr(), "a view keeps the buffer taken"
    del d, view
    e = kernels._kept_padded_buffer(cache, (2, 2, 4, 4), torch.int32, torch.device("cpu"))
    assert e.shape[0] == 2 and len(cache) == 1, "a new geometry replaces the buffer"


def test_hand_off_buffers_do_not_travel_with_copies_of_a_module():
    import copy
    import pickle
    conv = modules.Conv2dShift(4, 8, 3, padding=1)
    conv.__dict__["_handoff_buffers"] = {"k": torch.zeros(3)}
    clone = copy.deepcopy(conv)
    assert "_handoff_buffers" not in clone.__dict__ and "_handoff_buffers" in conv.__dict__
    assert torch.equal(clone.shift, conv.shift) and clone.shift_range == conv.shift_range
    again = pickle.loads(pickle.dumps(conv))
    assert "_handoff_buffers" not in again.__dict__ and torch.equal(again.sign, conv.sign)
    convq = modules_q.Conv2dShiftQ(4, 8, 3, padding=1)
    convq.__dict__["_handoff_buffers"] = {"k": torch.zeros(3)}
    assert "_handoff_buffers" not in copy.deepcopy(convq).__dict__
