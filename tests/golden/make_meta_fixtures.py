"""Writes tests/golden/meta/*.meta: engine sidecars produced by the reference's own JSON library
(oracle/_ref/meta_ref: nlohmann::json as vendored in the reference, driven call for call like
source/trt_engine/trt_common/trt_meta_data.cpp:81-97).  Needs `make -C oracle ref`, i.e. the
reference tree; the fixtures it writes are data and are committed, so the tests that read them run
anywhere.  CASES is also what the tests expect to read back."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
BIN = os.path.join(ROOT, "oracle", "_ref", "meta_ref")

# name -> (infer_mode, opt_batch_size, max_batch_size, unused_input_indices, output_indices, torch_module_path)
CASES = {
    "defaults": (0, -1, -1, [], [], ""),
    "dlrm_half": (1, 65536, 65536, [], [0], "dlrm.pth"),
    "bert_int8": (2, 16, 32, [3, 1], [2, 0, 1], "models/bert large \"v2\"\\final.pth"),
    "calib": (3, 1, 1, [0, 5, 7, 9], [4], "/abs/path/模型.pt"),
}


def main():
    os.makedirs(os.path.join(HERE, "meta"), exist_ok=True)
    for name, (mode, opt, mx, unused, outs, path) in CASES.items():
        dst = os.path.join(HERE, "meta", name + ".meta")
        subprocess.check_call([BIN, "write", dst, str(mode), str(opt), str(mx), ",".join(map(str, unused)),
                               ",".join(map(str, outs)), path])
        print(dst)


if __name__ == "__main__":
    main()
