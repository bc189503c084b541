"""Writes tests/golden/export_tiny/: two tiny checkpoints in the Boilerplate on-disk format, produced by the REFERENCE's
own exporter (boilerplate/format/export.py:115-300), so that the reader in deepseekternarized_amd/checkpoint.py is
checked against files it did not write itself.

Run in the build container only (the reference tree does not travel):

    python tests/golden/make_export_fixture.py [/root/reference]

What is written (data only: JSON + safetensors, a few KB each):

* ``source/``      the source checkpoint: config.json and weights.safetensors with six small bf16 expert weights
                   (two experts x w1 / w2 / w3, K = 200 so that the last scale group and the last packed byte are ragged)
                   and one weight that no rule matches (stays Mode A)
* ``mode_c_tq1/``  Mode C, k = 2 residual terms, TQ1, fp16 scales, group 128, act int8 (the exporter's defaults)
* ``mode_d_tq2/``  Mode D (one absmean term), TQ2, bf16 scales, group 64, act bf16
"""

from __future__ import annotations

import json
import shutil
import sys
from pathlib import Path

import torch
from safetensors.torch import save_file

HERE = Path(__file__).resolve().parent
OUT = HERE / "export_tiny"


def main() -> int:
    ref = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    sys.path.insert(0, str(ref))
    from boilerplate.format.export import export
    from boilerplate.format.policy import Policy

    if OUT.exists():
        shutil.rmtree(OUT)
    src = OUT / "source"
    src.mkdir(parents=True)
    g = torch.Generator().manual_seed(0)
    tensors = {}
    for e in range(2):
        for w, (n, k) in (("w1", (16, 200)), ("w3", (16, 200)), ("w2", (24, 160))):
            tensors[f"layers.0.ffn.experts.{e}.{w}.weight"] = (torch.randn(n, k, generator=g) * 0.05).to(torch.bfloat16)
    tensors["layers.0.attn.wq.weight"] = (torch.randn(8, 32, generator=g) * 0.05).to(torch.bfloat16)
    save_file(tensors, str(src / "weights.safetensors"))
    (src / "config.json").write_text(json.dumps({"model_type": "fixture", "dim": 200}))
    experts = r"experts\.\d+\.w[123]$"
    export(src, OUT / "mode_c_tq1", Policy.from_dict({"name": "c", "rules": [{"match": experts, "mode": "C", "k": 2, "packing": "tq1"}]}),
           log=lambda *a: None)
    export(src, OUT / "mode_d_tq2", Policy.from_dict({"name": "d", "rules": [{"match": experts, "mode": "D", "packing": "tq2", "group": 64,
                                                                               "scale_dtype": "bf16", "act": "bf16"}]}),
           log=lambda *a: None)
    for d in ("mode_c_tq1", "mode_d_tq2"):
        m = json.loads((OUT / d / "manifest.json").read_text())
        m["source"] = "source"  # (the exporter records the absolute path it was given)
        (OUT / d / "manifest.json").write_text(json.dumps(m, indent=1))
    print("wrote", OUT)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
