"""CompiledLogicNet: a trained network frozen into a flat netlist of arg-max gates and wiring, the
interface of the reference's src/difflogic/compiled_model.py (constructor, get_c_code, compile, load,
forward -> int32 [batch, classes]).

Two back ends:

* device="cuda": the netlist is evaluated by the packed-bit HIP kernels, 64 samples per word, without any
  nn.Module in the loop.  Beyond the reference, conv-logic blocks are part of the netlist (selection taps and
  7 gate ids per kernel), and the netlist can be written to / read from one .npz file (save / load_netlist).
* device="cpu": the reference's route -- C source with one expression per gate and bit-sliced adders for
  the per-class sums, compiled with gcc or clang into a shared object (fully connected networks only, as in
  the reference).
"""
import ctypes
import math
import shutil
import subprocess
import tempfile

import numpy as np
import torch

from ..hip import convlogic_hip, difflogic_hip
from .difflogic import GroupSum, LogicLayer
from .packbitstensor import PackBitsTensor

# the 16 two-input gates in the reference's numbering (src/difflogic/functional.py:7-24), as C expressions
GATE_EXPR = ("{z}", "{a} & {b}", "{a} & ~{b}", "{a}", "{b} & ~{a}", "{b}", "{a} ^ {b}", "{a} | {b}",
             "~({a} | {b})", "~({a} ^ {b})", "~{b}", "~{b} | {a}", "~{a}", "~{a} | {b}", "~({a} & {b})", "~{z}")
C_TYPE = {8: "signed char", 16: "short", 32: "int", 64: "long long"}
NP_TYPE = {8: np.int8, 16: np.int16, 32: np.int32, 64: np.int64}


def _is_conv(layer):
    from ..convlogic.convlogic_layer import ConvLogicLayer
    return isinstance(layer, ConvLogicLayer)


class CompiledLogicNet(torch.nn.Module):
    def __init__(self, model, device="cuda", num_bits=64, cpu_compiler="gcc", verbose=False):
        super().__init__()
        assert cpu_compiler in ("clang", "gcc"), cpu_compiler
        assert num_bits in (8, 16, 32, 64), num_bits
        assert device in ("cuda", "cpu"), device
        self.device, self.num_bits, self.cpu_compiler = device, num_bits, cpu_compiler
        self.lib_fn = None
        self.stages = []                 # ("conv", selection, gates, geometry) | ("fc", a, b, op, in_dim)
        self.num_inputs = self.num_classes = None
        if model is None:
            return
        layers = list(model.network) if hasattr(model, "network") else list(model)
        assert isinstance(layers[-1], GroupSum), f"The last layer of the model must be GroupSum, but it is {type(layers[-1])}."
        self.num_classes = layers[-1].k
        for layer in layers[:-1]:
            if isinstance(layer, LogicLayer):
                if self.num_inputs is None and not self.stages:
                    self.num_inputs = layer.in_dim
                self.stages.append(("fc", layer.indices_0.detach().cpu().numpy().astype(np.int64),
                                    layer.indices_1.detach().cpu().numpy().astype(np.int64),
                                    layer.weights.detach().argmax(-1).cpu().numpy().astype(np.uint8), int(layer.in_dim)))
            elif _is_conv(layer):
                assert layer.complete, "only complete conv-logic blocks can be compiled"
                geo = np.array([layer.in_channels, *layer.stride, *layer.padding, *layer.kernel], dtype=np.int64)
                self.stages.append(("conv", layer.selection.detach().cpu().numpy().astype(np.int32),
                                    layer.weights.detach().argmax(-1).cpu().numpy().astype(np.uint8), geo))
            elif isinstance(layer, torch.nn.Flatten):
                if verbose:
                    print("Flatten: layout change only")
            else:
                raise AssertionError(f"Error: layer {type(layer)} / {layer} unknown.")
        assert self.stages and self.stages[-1][0] == "fc", "the layer in front of GroupSum must be a LogicLayer"
        self.num_out_per_class = len(self.stages[-1][1]) // self.num_classes
        self._device_tables = None

    # ---- flat netlist file -----------------------------------------------------------------------
    def save(self, path):
        """One .npz file: stage kinds in order plus their integer tables."""
        blob = {"kinds": np.array([s[0] for s in self.stages]), "num_classes": np.int64(self.num_classes),
                "num_bits": np.int64(self.num_bits)}
        for i, s in enumerate(self.stages):
            if s[0] == "fc":
                blob[f"{i}_a"], blob[f"{i}_b"], blob[f"{i}_op"], blob[f"{i}_in"] = s[1], s[2], s[3], np.int64(s[4])
            else:
                blob[f"{i}_selection"], blob[f"{i}_gates"], blob[f"{i}_geometry"] = s[1], s[2], s[3]
        np.savez_compressed(path, **blob)

    @staticmethod
    def load_netlist(path, device="cuda"):
        z = np.load(path, allow_pickle=False)
        self = CompiledLogicNet(None, device=device, num_bits=int(z["num_bits"]))
        self.num_classes = int(z["num_classes"])
        for i, kind in enumerate(z["kinds"]):
            if str(kind) == "fc":
                self.stages.append(("fc", z[f"{i}_a"], z[f"{i}_b"], z[f"{i}_op"], int(z[f"{i}_in"])))
            else:
                self.stages.append(("conv", z[f"{i}_selection"], z[f"{i}_gates"], z[f"{i}_geometry"]))
        first = self.stages[0]
        self.num_inputs = first[4] if first[0] == "fc" else None
        self.num_out_per_class = len(self.stages[-1][1]) // self.num_classes
        self._device_tables = None
        return self

    # ---- GPU back end --------------------------------------------------------------------------
    def _tables(self, dev):
        if self._device_tables is None or self._device_tables[0] != dev:
            tabs = []
            for s in self.stages:
                if s[0] == "fc":
                    a, b = torch.from_numpy(s[1]).to(dev), torch.from_numpy(s[2]).to(dev)
                    tabs.append((a, b, torch.from_numpy(s[3]).to(dev), difflogic_hip.eval_plan(a, b, s[4])))
                else:
                    tabs.append((torch.from_numpy(s[1]).to(dev), torch.from_numpy(s[2]).to(dev).contiguous()))
            self._device_tables = (dev, tabs)
        return self._device_tables[1]

    def _forward_gpu(self, x):
        if isinstance(x, np.ndarray):
            x = torch.from_numpy(x)
        if not isinstance(x, PackBitsTensor):
            if not x.is_cuda:
                x = x.cuda()
            x = PackBitsTensor(x.bool(), 64)
        tabs = self._tables(x.t.device)
        for s, tab in zip(self.stages, tabs):
            if s[0] == "conv":
                assert x.image and x.t.shape[1] == int(s[3][0]), (x.image, tuple(x.t.shape), int(s[3][0]))
                x.t = convlogic_hip.full_convlogic_eval_packed(x.t.contiguous(), tab[1], tab[0], *(int(v) for v in s[3][1:]))
            else:
                x.flatten()
                assert x.t.shape[0] == s[4], (tuple(x.t.shape), s[4])
                x.t = difflogic_hip.eval_planned(x.t, tab[0], tab[1], tab[2], tab[3])
        return x.group_sum(self.num_classes)

    # ---- CPU back end: generated C -----------------------------------------------------------
    def _fc_only(self):
        assert all(s[0] == "fc" for s in self.stages), "C code is generated for fully connected networks only"
        return [(s[1], s[2], s[3]) for s in self.stages]

    def get_gate_code(self, var1, var2, gate_op):
        """C expression of gate `gate_op` on two words (bitwise twins of the 16 relaxed operations)."""
        expr = GATE_EXPR[int(gate_op)].format(a=var1, b=var2, z=f"(({C_TYPE[self.num_bits]})0)")
        return f"({C_TYPE[self.num_bits]})({expr})" if self.num_bits < 32 else expr

    def get_c_code(self):
        """Straight-line C: `logic_gate_net(inp, out)` evaluates one word per feature; `apply_logic_gate_net(inp,
        out, len)` packs `len` groups of num_bits bool samples [sample, feature] (sample s of a group -> bit s),
        runs the net and counts the set output bits per class with ripple adders over bit planes; out is int
        [sample, class]."""
        layers = self._fc_only()
        word, bits = C_TYPE[self.num_bits], self.num_bits
        uword = "unsigned " + word.replace("signed ", "")
        last = len(layers) - 1
        lines = ["#include <stddef.h>", "#include <stdlib.h>", "#include <stdbool.h>", "",
                 f"void logic_gate_net({word} const *inp, {word} *out) {{"]
        for li, (a, b, op) in enumerate(layers):
            for j, (ja, jb, jo) in enumerate(zip(a, b, op)):
                va = f"inp[{ja}]" if li == 0 else f"v{li - 1}_{ja}"
                vb = f"inp[{jb}]" if li == 0 else f"v{li - 1}_{jb}"
                target = f"out[{j}]" if li == last else f"const {word} v{li}_{j}"
                lines.append(f"\t{target} = {self.get_gate_code(va, vb, jo)};")
        lines.append("}")
        n_in, n_out, k = self.num_inputs, len(layers[-1][0]), self.num_classes
        per = n_out // k
        planes = max(1, math.ceil(math.log2(per + 1)))
        lines.append(f"""
void apply_logic_gate_net(bool const *inp, int *out, size_t len) {{
    {word} *packed = malloc({n_in} * sizeof({word}));
    {word} *res = malloc({n_out} * sizeof({word}));
    {uword} plane[{planes}];
    for (size_t i = 0; i < len; ++i) {{
        const bool *grp = inp + i * {bits} * {n_in};
        for (size_t d = 0; d < {n_in}; ++d) {{
            {uword} w = 0;
            for (size_t s = 0; s < {bits}; ++s) w |= ({uword})(grp[s * {n_in} + d] != 0) << s;
            packed[d] = ({word})w;
        }}
        logic_gate_net(packed, res);
        for (size_t c = 0; c < {k}; ++c) {{
            for (int d = 0; d < {planes}; ++d) plane[d] = 0;
            for (size_t a = 0; a < {per}; ++a) {{
                {uword} carry = ({uword})res[c * {per} + a];
                for (int d = 0; d < {planes}; ++d) {{
                    const {uword} t = plane[d];
                    plane[d] = t ^ carry;
                    carry &= t;
                }}
            }}
            for (size_t s = 0; s < {bits}; ++s) {{
                int count = 0;
                for (int d = 0; d < {planes}; ++d) count |= (int)((plane[d] >> s) & 1) << d;
                out[(i * {bits} + s) * {k} + c] = count;
            }}
        }}
    }}
    free(packed);
    free(res);
}}
""")
        return "\n".join(lines)

    def compile(self, opt_level=1, save_lib_path=None, verbose=False):
        """Builds the generated C into a shared object and binds `apply_logic_gate_net` (device="cpu")."""
        assert self.device == "cpu", f"Device {self.device} needs no compilation."
        code = self.get_c_code()
        with tempfile.TemporaryDirectory() as tmp:
            src, lib = f"{tmp}/net.c", f"{tmp}/net.so"
            with open(src, "w") as f:
                f.write(code)
            if verbose:
                print(f"C code has {code.count(chr(10)) + 1} lines")
            res = subprocess.run([self.cpu_compiler, "-shared", "-fPIC", f"-O{opt_level}", "-o", lib, src], capture_output=True, text=True)
            if res.returncode != 0:
                raise RuntimeError(f"compilation exited with error code {res.returncode}\n{res.stderr}")
            if save_lib_path is not None:
                shutil.copy(lib, save_lib_path)
            self.lib_fn = self._bind(lib)

    @staticmethod
    def _bind(path):
        fn = ctypes.cdll.LoadLibrary(path).apply_logic_gate_net
        fn.restype = None
        fn.argtypes = [np.ctypeslib.ndpointer(ctypes.c_bool, flags="C_CONTIGUOUS"),
                       np.ctypeslib.ndpointer(ctypes.c_int32, flags="C_CONTIGUOUS"), ctypes.c_size_t]
        return fn

    @staticmethod
    def load(save_lib_path, num_classes, num_bits):
        """Binds a shared object written by compile(save_lib_path=...)."""
        self = CompiledLogicNet(None, device="cpu", num_bits=num_bits)
        self.num_classes = num_classes
        self.lib_fn = CompiledLogicNet._bind(save_lib_path)
        return self

    def _forward_cpu(self, x):
        assert self.lib_fn is not None, "call compile() (or load()) first"
        x = x.cpu().numpy() if isinstance(x, torch.Tensor) else np.asarray(x)
        x = np.ascontiguousarray(x.reshape(x.shape[0], -1).astype(np.bool_))
        groups = math.ceil(x.shape[0] / self.num_bits)
        pad = groups * self.num_bits - x.shape[0]
        if pad:
            x = np.concatenate([x, np.zeros((pad, x.shape[1]), dtype=np.bool_)])
        out = np.zeros(x.shape[0] * self.num_classes, dtype=np.int32)
        self.lib_fn(x.reshape(-1), out, groups)
        out = torch.from_numpy(out).view(groups * self.num_bits, self.num_classes)
        return out[:out.shape[0] - pad] if pad else out

    def forward(self, x, verbose=False):
        """bool [batch, features] (or [batch, C, H, W] for networks that start with conv blocks) -> int32
        [batch, classes]: per-class counts of set output bits, i.e. GroupSum without the division by tau."""
        return self._forward_gpu(x) if self.device == "cuda" else self._forward_cpu(x)
