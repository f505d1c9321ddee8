"""Writes tests/golden/cogvideox_tuned_params.json from the tuned-parameter file the reference ships.

Run once in a container that has the reference checkout (never on the GPU box):

    python tests/golden/make_tuned_params_fixture.py [/root/reference]

The source, evaluate/models_dict/CogVideoX-2b_0.06_0.07.pt, is a plain state dict written by
extract_sparse_attention_state_dict (spas_sage_attn/autotune.py:28-38): 30 transformer blocks x 5 tensors of shape
(30,) (is_sparse bool; cdfthreshd, simthreshd1, simthreshd2, pvthreshd float32).  It is read with
torch.load(weights_only=True), which executes nothing from the file.  The JSON keeps every float32 exactly
(Python floats print round-trip) and is data only.
"""
import json
import os
import sys

import torch


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    sd = torch.load(os.path.join(ref, "evaluate", "models_dict", "CogVideoX-2b_0.06_0.07.pt"), weights_only=True,
                    map_location="cpu")
    out = {}
    for key, t in sd.items():
        out[key] = {"dtype": str(t.dtype).replace("torch.", ""), "values": [v for v in t.tolist()]}
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cogvideox_tuned_params.json")
    with open(dst, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print(dst, len(out), "tensors")


if __name__ == "__main__":
    main()
