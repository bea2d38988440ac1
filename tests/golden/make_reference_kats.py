"""Writes ``reference_kats.json``: the known-answer inputs the reference's own unit tests hold
for the embedding-bag path.

Tables are the raw little-endian float32 payloads stored inside the reference's TorchScript
archives (plain zip members; nothing is unpickled or executed); ids and offsets are the literals
of the tests that use those archives:

  data/torch_unit_tests/nodes/embedding_bag.pth   + source/unit_test/test_torch_nodes.h:178-185
  data/torch_unit_tests/dlrm.pth                  + source/unit_test/test_torch_dlrm.h:34-57
  data/torch_unit_tests/nodes/layer_norm_with_weights.pth + source/unit_test/test_torch_nodes.h:293-299

Run in the build container only (needs /root/reference):  python tests/golden/make_reference_kats.py
"""
import json
import os
import zipfile

import numpy as np

REF = "/root/reference/data/torch_unit_tests/"
HERE = os.path.dirname(os.path.abspath(__file__))


def member(path, name, shape):
    with zipfile.ZipFile(REF + path) as z:
        raw = z.read(name)
    return np.frombuffer(raw, "<f4").reshape(shape)


def main():
    kats = {}
    w = member("nodes/embedding_bag.pth", "embedding_bag/data/0", (5, 4))
    kats["embedding_bag_module"] = {
        "source": "test_torch_nodes.h:178-185, nodes/embedding_bag.pth",
        "table": w.tolist(), "mode": "sum",
        "indices": [1, 0, 3, 1, 4], "offsets": [0, 0, 0, 0, 0],
    }
    # dlrm.pth: tensors/2,3,4 are the three embedding tables (4x2, 3x2, 2x2), model.json names them.
    tables = [member("dlrm.pth", "dlrm/tensors/%d" % i, s) for i, s in ((2, (4, 2)), (3, (3, 2)), (4, (2, 2)))]
    kats["dlrm"] = {
        "source": "test_torch_dlrm.h:34-57, dlrm.pth",
        "mode": "sum",
        "tables": [t.tolist() for t in tables],
        "indices": [[3, 0, 2], [1, 1, 2], [1, 1]],
        "offsets": [[0, 1], [0, 1], [0, 1]],
    }
    g = member("nodes/layer_norm_with_weights.pth", "layer_norm_with_weights/data/0", (10,))
    b = member("nodes/layer_norm_with_weights.pth", "layer_norm_with_weights/data/1", (10,))
    kats["layer_norm_with_weights"] = {
        "source": "test_torch_nodes.h:293-299, nodes/layer_norm_with_weights.pth",
        "input_shape": [20, 5, 10], "ld": 10, "eps": 1e-5,
        "data0": g.tolist(), "data1": b.tolist(),
    }
    with open(os.path.join(HERE, "reference_kats.json"), "w") as f:
        json.dump(kats, f, indent=1)
    print(json.dumps(kats, indent=1)[:1500])


if __name__ == "__main__":
    main()
