"""Writes tests/golden/wiring_golden.json: seeded wiring / tap-selection vectors.

Only the RNG call order of the reference constructors cannot be pinned by a
closed form, so only these constructors are executed here (in the build
container, never on the GPU box):
  * difflogic.LogicLayer.__init__ -> get_connections (src/difflogic/difflogic.py:20-90,169-185)
  * difflogic.functional.get_unique_connections       (src/difflogic/functional.py:77-125)
  * ConvLogicLayer.__init__ -> generate_selection      (src/convlogic/convlogic_layer.py:94-160,377-452)
The output is data only: seeds, constructor arguments and the resulting integer
buffers (plus a float checksum of the logits drawn before them).

Usage:  python tests/golden/make_golden.py /root/reference
"""
import importlib.util
import json
import os
import sys

import torch


def main(ref_root):
    sys.path.insert(0, os.path.join(ref_root, "src"))
    from difflogic.difflogic import LogicLayer  # noqa: E402

    spec = importlib.util.spec_from_file_location(
        "ref_convlogic_layer", os.path.join(ref_root, "src", "convlogic", "convlogic_layer.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    ConvLogicLayer = mod.ConvLogicLayer

    out = {"torch_version": torch.__version__, "logic_layer": [], "conv_layer": []}

    for seed, in_dim, out_dim, conn in [
        (0, 12, 16, "random"), (1, 8, 8, "random"), (2, 64, 64, "random"), (3, 100, 50, "random"),
        (4, 30, 77, "random"), (0, 12, 16, "unique"), (5, 9, 20, "unique"), (6, 64, 32, "unique"),
    ]:
        torch.manual_seed(seed)
        layer = LogicLayer(in_dim, out_dim, implementation="python", connections=conn)
        out["logic_layer"].append({
            "seed": seed, "in_dim": in_dim, "out_dim": out_dim, "connections": conn,
            "indices_0": layer.indices_0.tolist(), "indices_1": layer.indices_1.tolist(),
            "weights_sum": float(layer.weights.double().sum()),
        })

    for seed, cin, cout, kernel, groups, complete in [
        (0, 3, 8, 3, 1, True), (1, 1, 32, 3, 1, True), (2, 9, 64, 3, 1, True), (3, 4, 6, 5, 1, False),
        (4, 6, 12, 3, 3, True), (5, 2, 5, (2, 4), 1, False), (6, 7, 9, 3, 2, True),
    ]:
        torch.manual_seed(seed)
        layer = ConvLogicLayer(cin, cout, kernel=kernel, groups=groups, complete=complete,
                               implementation="python")
        out["conv_layer"].append({
            "seed": seed, "in_channels": cin, "out_channels": cout, "kernel": kernel, "groups": groups,
            "complete": complete, "selection": layer.selection.tolist(),
            "weights_sum": float(layer.weights.double().sum()),
        })

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "wiring_golden.json")
    with open(path, "w") as f:
        json.dump(out, f)
    print("wrote", path)


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
