"""CPU-only tests: the C-ABI library loads and exports every declared symbol, the host-side python
backend agrees with the oracle, wiring matches the golden vectors, argument validation raises."""
import os
import re

import numpy as np
import pytest
import torch

import convlogic_amd as C
from convlogic_amd.difflogic import functional as Fn
from convlogic_amd.difflogic.difflogic import _reverse_wiring
from convlogic_amd.hip import _lib
from oracle import convlogic_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "convlogic_amd.h")).read()
    declared = set(re.findall(r"\b(clg_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.clg_abi_version() == 1
    assert lib.clg_last_error() == b""


def test_ctypes_signatures_match_the_header_prototypes():
    # every prototype of the header, argument by argument, against the ctypes declaration that calls it: a pointer
    # passed where the library reads an int64 (or an argument too few) would not fail at load time
    import ctypes
    header = open(os.path.join(ROOT, "include", "convlogic_amd.h")).read()
    header = re.sub(r"/\*.*?\*/", " ", header, flags=re.S)              # comments, also the ones inside argument lists
    header = re.sub(r"//[^\n]*", " ", header)
    protos = re.findall(r"\b(const char \*|int64_t|int|void)\s*(clg_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", header)
    assert {name for _, name, _ in protos} == set(_lib.SIGNATURES)

    def ctype_of(decl):
        decl = " ".join(decl.split())
        if decl == "void":
            return None
        if "*" in decl:
            return _lib._GP if "clg_conv_geom" in decl else ctypes.c_void_p
        base = decl.rsplit(" ", 1)[0] if " " in decl else decl        # drop the parameter name
        return {"int": ctypes.c_int, "int64_t": ctypes.c_int64, "double": ctypes.c_double}[base.replace("const ", "")]

    results = {"const char *": ctypes.c_char_p, "int64_t": ctypes.c_int64, "int": ctypes.c_int, "void": None}
    for ret, name, args in protos:
        want = [t for t in (ctype_of(a) for a in args.split(",")) if t is not None]
        res, got = _lib.SIGNATURES[name]
        assert res is results[ret], name
        assert len(got) == len(want), (name, len(got), len(want))
        for k, (g, w) in enumerate(zip(got, want)):
            assert g is w, (name, k, g, w)


def test_c_abi_rejects_bad_arguments_without_gpu():
    lib = _lib.load()
    assert lib.clg_fc_forward(7, 0, 0, 0, 0, 0, 4, 4, 4, None) == -1
    assert b"dtype" in lib.clg_last_error()
    assert lib.clg_group_bit_sum(8, 1, 1, 10, 4, 0, 3, None) == -1
    assert b"divisible" in lib.clg_last_error()
    assert lib.clg_pack_bits(1, 1, 4, 4, 12, None) == -1
    assert b"bit_count" in lib.clg_last_error()
    g = _lib.ConvGeom(1, 1, 5, 5, 1, 1, 1, 0, 0, 3, 3)    # conv output 3x3: odd
    import ctypes
    assert lib.clg_convblock_forward(0, ctypes.byref(g), 1, 1, 1, 1, 1, None) == -1
    assert b"divisible by 2" in lib.clg_last_error()


def test_missing_library_fails_loudly_and_product_never_imports_the_oracle(monkeypatch):
    # no silent fallback: without the built library the "cuda" implementation raises, naming the build step
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", os.path.join(ROOT, "convlogic_amd", "no_such_library.so"))
    assert not _lib.available()
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load()
    # and nothing under the package imports, opens or names the oracle
    for folder, _, files in os.walk(os.path.join(ROOT, "convlogic_amd")):
        for name in files:
            if name.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(folder, name)).read()
                assert "oracle" not in text, os.path.join(folder, name)


@pytest.mark.parametrize("i", range(16))
def test_bin_op_matches_oracle(i):
    a, b = torch.rand(20, dtype=torch.float64), torch.rand(20, dtype=torch.float64)
    assert torch.allclose(Fn.bin_op(a, b, i), O.bin_op(a, b, i), atol=1e-14)


def test_bin_op_s_matches_oracle():
    torch.manual_seed(0)
    a, b = torch.rand(5, 7, dtype=torch.float64), torch.rand(5, 7, dtype=torch.float64)
    w = torch.softmax(torch.randn(7, 16, dtype=torch.float64), -1)
    assert torch.allclose(Fn.bin_op_s(a, b, w), O.bin_op_s(a, b, w), atol=1e-14)


def test_wiring_golden(golden):
    for r in golden["logic_layer"]:
        torch.manual_seed(r["seed"])
        layer = C.LogicLayer(r["in_dim"], r["out_dim"], implementation="python", connections=r["connections"])
        assert layer.indices_0.tolist() == r["indices_0"] and layer.indices_1.tolist() == r["indices_1"]
        assert abs(float(layer.weights.detach().double().sum()) - r["weights_sum"]) < 1e-9
    for r in golden["conv_layer"]:
        torch.manual_seed(r["seed"])
        layer = C.ConvLogicLayer(r["in_channels"], r["out_channels"], kernel=r["kernel"], groups=r["groups"],
                                 complete=r["complete"], implementation="python")
        assert layer.selection.tolist() == r["selection"] and layer.selection.dtype == torch.int32
        assert abs(float(layer.weights.detach().double().sum()) - r["weights_sum"]) < 1e-9


def test_reverse_wiring_matches_oracle_loop():
    torch.manual_seed(1)
    idx0, idx1 = torch.randint(0, 9, (14,)), torch.randint(0, 9, (14,))
    idx1[3] = idx0[3]                                  # a self-paired neuron
    s1, f1 = _reverse_wiring(idx0.numpy(), idx1.numpy(), 9)
    s2, f2 = O.csr_build(idx0, idx1, 9)
    assert torch.equal(s1, s2) and torch.equal(f1, f2)


def test_logic_layer_python_matches_oracle():
    torch.manual_seed(2)
    layer = C.LogicLayer(10, 12, implementation="python")
    x = torch.rand(4, 10)
    y = layer(x)
    want = O.logic_fc_forward(x, layer.indices_0, layer.indices_1, O.gate_weights(layer.weights, True))
    assert torch.allclose(y, want, atol=1e-6)
    layer.eval()
    xb = torch.randint(0, 2, (4, 10)).float()
    yb = layer(xb)
    assert torch.all((yb == 0) | (yb == 1))
    assert torch.equal(yb, O.logic_fc_forward(xb, layer.indices_0, layer.indices_1, O.gate_weights(layer.weights, False)))


@pytest.mark.parametrize("stride,pad,kernel", [(1, 1, 3), (2, 2, 4), (1, 0, 3)])
def test_conv_layer_python_matches_oracle(stride, pad, kernel):
    torch.manual_seed(3)
    layer = C.ConvLogicLayer(3, 4, stride=stride, padding=pad, kernel=kernel, implementation="python", complete=True)
    x = torch.randn(2, 3, 8, 8)
    y = layer(x)
    want = O.conv_block_forward(x, O.gate_weights(layer.weights, True), layer.selection, (stride,) * 2, (pad,) * 2, (kernel,) * 2)
    assert y.shape == want.shape and torch.allclose(y, want, atol=1e-6)
    split = C.ConvLogicLayer(3, 4, stride=stride, padding=pad, kernel=kernel, implementation="python", selection=layer.selection)
    y4 = split(x)
    want4 = O.conv4_forward(x, O.gate_weights(split.weights, True), layer.selection, (stride,) * 2, (pad,) * 2, (kernel,) * 2)
    assert torch.allclose(y4, want4, atol=1e-6)


def test_tree_layer_python_all_gates():
    layer = C.TreeLogicLayer(channels=16, input_bits=8, implementation="python")
    logits = torch.full((16, 4, 16), float("-inf"))
    for g in range(16):
        logits[g, :, g] = 0.0
    with torch.no_grad():
        layer.weights.copy_(logits)
    flat = [0.0, 0.0, 0.0, 1.0, 1.0, 0.0, 1.0, 1.0]
    x = torch.tensor(flat).reshape(1, 1, 1, 1, 8).expand(-1, 16, -1, -1, -1)
    a, b = torch.tensor(flat[::2]), torch.tensor(flat[1::2])
    want = torch.stack([O.bin_op(a, b, g) for g in range(16)]).view(1, 16, 1, 1, 4)
    assert torch.equal(layer(x), want)


def test_pool_layer_and_errors():
    x = torch.randn(2, 3, 8, 8)
    assert torch.equal(C.PoolLogicLayer()(x), torch.nn.functional.max_pool2d(x, 2, 2))
    assert torch.equal(C.PoolLogicLayer()(x.unsqueeze(-1)), torch.nn.functional.max_pool2d(x, 2, 2))
    with pytest.raises(ValueError):
        C.PoolLogicLayer()(torch.randn(1, 2, 3))
    with pytest.raises(ValueError):
        C.PoolLogicLayer()(torch.randn(1, 1, 1, 4, 2))


def test_group_sum_and_grad_factor():
    x = torch.rand(3, 20, requires_grad=True)
    y = C.GroupSum(5, tau=2.0)(C.GradFactor.apply(x, 3.0))
    assert torch.allclose(y, O.group_sum(x.detach(), 5, 2.0))
    y.sum().backward()
    assert torch.allclose(x.grad, torch.full_like(x, 1.5))


def test_constructor_validation():
    with pytest.raises(AssertionError):
        C.LogicLayer(10, 4, implementation="python")          # fewer than in_dim/2 neurons
    with pytest.raises(AssertionError):
        C.LogicLayer(4, 4, implementation="tpu")
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError):
            C.ConvLogicLayer(1, 1, implementation="cuda")
        with pytest.raises(NotImplementedError):
            C.PackBitsTensor(torch.zeros(4, 4, dtype=torch.bool))
    layer = C.ConvLogicLayer(2, 3, residual_init=True, complete=True, implementation="python")
    assert torch.all(layer.weights.argmax(-1) == 3)
    assert set(layer.state_dict()) == {"weights", "selection"}
    fc = C.LogicLayer(4, 4, implementation="python")
    assert set(fc.state_dict()) == {"weights", "indices_0", "indices_1"}


def test_one_by_one_kernel_raises_instead_of_redrawing_forever():
    # the reference redraws only (row, column) of the second tap of a pair (src/convlogic/convlogic_layer.py:437-448): with a
    # window of one element its loop never ends once both taps drew the same channel; this package raises
    torch.manual_seed(0)
    with pytest.raises(ValueError):
        C.ConvLogicLayer(8, 5, kernel=1, padding=0, implementation="python")


def test_bad_selection_and_wiring_raise_on_the_host():
    # a tap outside the input channels / receptive field, or a wiring index outside the input features, would be an
    # out-of-range access inside a kernel: both are rejected on the host (ValueError), also after in-place edits
    good = C.ConvLogicLayer(2, 3, kernel=3, implementation="python").selection
    for bad_tap in ((5 << 16) | (1 << 8) | 1, (1 << 16) | (3 << 8) | 1, (1 << 16) | (1 << 8) | 7):
        bad = good.clone()
        bad[1, 4] = bad_tap
        with pytest.raises(ValueError, match="selection names a tap outside"):
            C.ConvLogicLayer(2, 3, kernel=3, selection=bad, implementation="python")
    with pytest.raises(ValueError, match="int32"):
        C.ConvLogicLayer(2, 3, kernel=3, selection=good.long(), implementation="python")
    layer = C.ConvLogicLayer(2, 3, kernel=3, selection=good.clone(), implementation="python")
    layer._check_selection()
    layer.selection[0, 0] = 9 << 16                              # in-place edit: seen through the version counter
    with pytest.raises(ValueError):
        layer._check_selection()
    layer.selection.data[0, 0] = good[0, 0]                      # .data writes bypass it ...
    layer.invalidate()                                            # ... and need an explicit invalidate()
    layer._check_selection()

    fc = C.LogicLayer(6, 8, implementation="python")
    fc._check_wiring()
    fc.indices_1[3] = 6
    with pytest.raises(ValueError, match="indices_1"):
        fc._check_wiring()
    fc.indices_1[3] = 0
    fc._check_wiring()
    fc.indices_0[0] = -1
    with pytest.raises(ValueError, match="indices_0"):
        fc._check_wiring()
    # load_state_dict re-arms the checks
    fc2 = C.LogicLayer(6, 8, implementation="python")
    fc2._check_wiring()
    fc2.load_state_dict(fc.state_dict())
    with pytest.raises(ValueError):
        fc2._check_wiring()


# ---- model topologies -----------------------------------------------------------------------------
def test_model_topologies_layers_keys_and_shapes():
    # src/convlogic/model.py:16-58 and :68-106: layer order, widths and state_dict names
    torch.manual_seed(0)
    m = C.ConvLogicMnistModel(k_param=2, implementation="python")
    kinds = [type(l).__name__ for l in m.network]
    assert kinds == ["ConvLogicLayer"] * 3 + ["Flatten"] + ["LogicLayer"] * 3 + ["GroupSum"]
    assert [(l.in_channels, l.out_channels, l.kernel, l.padding) for l in m.network[:3]] == \
        [(1, 2, (5, 5), (0, 0)), (2, 6, (3, 3), (1, 1)), (6, 18, (3, 3), (1, 1))]
    assert [(l.in_dim, l.out_dim) for l in m.network[4:7]] == [(162, 2560), (2560, 1280), (1280, 640)]
    assert m.network[7].k == 10 and m.network[7].tau == 6.5
    keys = list(m.state_dict())
    assert keys[:2] == ["network.0.weights", "network.0.selection"]
    assert "network.4.indices_0" in keys and "network.4.indices_1" in keys
    assert m(torch.rand(3, 1, 28, 28)).shape == (3, 10)
    # residual init: gate 3 ("A") carries p = e^5 / (e^5 + 15)
    p = torch.softmax(m.network[0].weights, -1)[0, 0]
    assert abs(p[3].item() - 0.908208) < 1e-5

    c = C.ConvLogicCifarModel(k_param=2, input_channels=3, implementation="python")
    assert [(l.in_channels, l.out_channels) for l in c.network[:4]] == [(3, 2), (2, 8), (8, 32), (32, 64)]
    assert [(l.in_dim, l.out_dim) for l in c.network[5:8]] == [(256, 2560), (2560, 1280), (1280, 640)]
    assert c.extra_layers == 1 and c.network[8].tau == 20
    assert c(torch.rand(2, 3, 32, 32)).shape == (2, 10)


def test_model_construction_draws_like_the_layers_in_order():
    # equal seeds give equal parameters whether the layers are built by the model or by hand in its order
    torch.manual_seed(5)
    m = C.ConvLogicMnistModel(k_param=1, implementation="python")
    torch.manual_seed(5)
    first = C.ConvLogicLayer(1, 1, kernel=5, padding=0, residual_init=True, complete=True, implementation="python")
    second = C.ConvLogicLayer(1, 3, kernel=3, padding=1, residual_init=True, complete=True, implementation="python")
    assert torch.equal(m.network[0].selection, first.selection) and torch.equal(m.network[1].selection, second.selection)


# ---- CompiledLogicNet: generated C (the reference's CPU route) -------------------------------------
@pytest.mark.parametrize("bits", [8, 64])
def test_compiled_net_c_code_matches_eval_forward(bits, tmp_path):
    # src/difflogic/compiled_model.py: forward(bool [N, F]) -> int32 [N, classes] = GroupSum counts of the
    # eval-mode network; compared with this package's torch-op ("python") implementation on binary inputs
    from convlogic_amd.difflogic import CompiledLogicNet
    torch.manual_seed(bits)
    dims = [12, 24, 18, 12]
    model = torch.nn.Sequential(torch.nn.Flatten(), *[C.LogicLayer(a, b, implementation="python") for a, b in zip(dims, dims[1:])],
                                C.GroupSum(3, tau=4.0)).eval()
    with torch.no_grad():
        for m in model:
            if hasattr(m, "weights"):
                m.weights.copy_(torch.randn_like(m.weights))
    net = CompiledLogicNet(model, device="cpu", num_bits=bits)
    assert net.num_inputs == 12 and net.num_classes == 3 and net.num_out_per_class == 4
    code = net.get_c_code()
    assert "void logic_gate_net(" in code and "void apply_logic_gate_net(bool const *inp, int *out, size_t len)" in code
    lib = tmp_path / "net.so"
    net.compile(save_lib_path=str(lib))
    x = torch.randint(0, 2, (bits + 5, 12)).bool()                 # ragged last group
    want = torch.round(model(x.float()) * 4.0).to(torch.int32)
    assert torch.equal(net(x), want)
    again = CompiledLogicNet.load(str(lib), num_classes=3, num_bits=bits)
    assert torch.equal(again(x.numpy()), want)


def test_compiled_net_gate_expressions_are_the_truth_tables():
    from convlogic_amd.difflogic.compiled_model import GATE_EXPR
    for i, expr in enumerate(GATE_EXPR):
        for a in (0, 1):
            for b in (0, 1):
                got = eval(expr.format(a=-a, b=-b, z="0")) & 1       # all-ones / all-zeros words
                assert got == (i >> (3 - 2 * a - b)) & 1, (i, a, b)


def test_compiled_net_netlist_file_round_trip(tmp_path):
    from convlogic_amd.difflogic import CompiledLogicNet
    torch.manual_seed(1)
    m = C.ConvLogicMnistModel(k_param=1, implementation="python")
    net = CompiledLogicNet(m, device="cuda")
    assert [s[0] for s in net.stages] == ["conv"] * 3 + ["fc"] * 3 and net.num_classes == 10
    path = tmp_path / "net.npz"
    net.save(str(path))
    back = CompiledLogicNet.load_netlist(str(path))
    assert len(back.stages) == 6 and back.num_classes == 10
    for s, t in zip(net.stages, back.stages):
        assert s[0] == t[0] and all(np.array_equal(np.asarray(u), np.asarray(v)) for u, v in zip(s[1:], t[1:]))


def test_recorded_traffic_file_feeds_the_bench_line():
    # bench.py reports `roofline.traffic` from profiles/traffic.json (recorded rocprofv3 counters): the file names the
    # commit of every measurement and the method, and holds the entries bench.py asks for; a missing entry reads as None, never as a guess
    import json
    import bench
    with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
        rec = json.load(f)
    assert "rocprofv3 --pmc FETCH_SIZE" in rec["method"] and all(w["commit"] for w in rec["workloads"].values())
    assert bench._traffic("c2", "eval_packed_walk_kernel_bytes_per_launch") == rec["workloads"]["c2"]["eval_packed_walk_kernel_bytes_per_launch"]
    for wl in ("c4", "c3", "c1", "c5"):
        got = bench._traffic(wl, "step_bytes")
        assert got == rec["workloads"][wl]["step_bytes"] and got > 0
        assert abs(sum(k["bytes_per_launch"] * k["launches_per_step"] for k in rec["workloads"][wl]["kernels"].values()) - got) <= len(rec["workloads"][wl]["kernels"])
    assert bench._traffic("c9", "step_bytes") is None and bench._traffic("c4", "no_such_key") is None


def test_python_path_rejects_an_index_rewired_out_of_range_through_data():
    # the torch-op backend indexes with the wiring on every call (as the reference does, src/difflogic/difflogic.py:149-164):
    # an index written through `.data` past the version counter raises there; the HIP kernels force it into range instead
    # (tests/test_gpu_fc.py::test_fc_index_corrupted_behind_the_host_check_is_clamped_not_faulting)
    import pytest
    layer = C.LogicLayer(8, 12, implementation="python")
    x = torch.rand(4, 8)
    layer(x)
    layer.indices_0.data[3] = 8
    with pytest.raises((IndexError, RuntimeError)):
        layer(x)
