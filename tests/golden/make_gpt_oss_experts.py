"""Writes tests/golden/tiny_gpt_oss/: the MXFP4 expert tensors of the reference's tiny gpt-oss fixture, as data.

    python tests/golden/make_gpt_oss_experts.py [/root/reference]

The reference keeps a four-layer gpt-oss store under tests/fixtures/tiny_gpt_oss (random MXFP4 bytes per expert:
`mlp.experts.{gate_up,down}_proj_{blocks,scales}` and the experts' bf16 biases, written by its tests/make_fixtures.py).
Only those tensors, the router's weight and bias beside them and the config's shape fields are copied - through safetensors, nothing of the reference is
run - into one shard with an index, which is all the MXFP4 store reader (btb_amd/load.py: `load_mx_experts`) needs.
"""

from __future__ import annotations

import glob
import json
import os
import sys

from safetensors import safe_open
from safetensors.torch import save_file

HERE = os.path.dirname(os.path.abspath(__file__))


def main(ref: str) -> None:
    src = os.path.join(ref, "tests", "fixtures", "tiny_gpt_oss")
    out = os.path.join(HERE, "tiny_gpt_oss")
    os.makedirs(out, exist_ok=True)
    keep = {}
    for shard in sorted(glob.glob(os.path.join(src, "*.safetensors"))):
        with safe_open(shard, framework="pt") as f:
            for k in f.keys():
                if ".mlp.experts." in k and k.endswith(("_blocks", "_scales", "_bias")) \
                        or k.endswith(("mlp.router.weight", "mlp.router.bias")):
                    keep[k] = f.get_tensor(k).contiguous()
    name = "experts-00001-of-00001.safetensors"
    save_file(keep, os.path.join(out, name))
    with open(os.path.join(out, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": {k: name for k in sorted(keep)}}, f, indent=1)
    with open(os.path.join(src, "config.json")) as f:
        cfg = json.load(f)
    fields = ("model_type", "hidden_size", "intermediate_size", "num_hidden_layers", "num_local_experts",
              "num_experts_per_tok", "experts_per_token", "swiglu_limit")
    with open(os.path.join(out, "config.json"), "w") as f:
        json.dump({k: cfg[k] for k in fields if k in cfg}, f, indent=1)
    print(f"{len(keep)} tensors -> {out}")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
