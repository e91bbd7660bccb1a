#!/usr/bin/env python3
"""Import the reference's committed test DATA as compact golden fixtures.

Reads (as data, nothing is imported or executed):
  NNtrain.Core.Tests/Fixtures/QwenGgufReference/reference.gguf   (gguf-py written GGUF v3, 6 tensors)
  NNtrain.Core.Tests/Fixtures/QwenGgufReference/expected.json    (gguf-py decoded values + float64 linear)
  NNtrain.Core.Tests/Fixtures/IqQuantReference/iq-quant-blocks.json  (native ggml decode of 139 blocks)
and writes, beside this script:
  qwen_gguf_reference.gguf   byte copy of the GGUF tensor fixture
  qwen_gguf_expected.json    byte copy of its manifest
  iq_quant_blocks.json       the 139 block cases re-serialised compactly: decoded float32 values as
                             base64 of their little-endian bytes instead of a JSON number list
  LICENSE.llama.cpp          MIT notice that accompanies the native-ggml fixture

The per-case sha256 of the decoded bytes recorded by the reference is re-checked while converting, so
the compact form is proven to hold exactly the float32 bits the reference's tests compare against
(NNtrain.Core.Tests/Qwen35GpuIqTests.cs:25-45, QwenGgufIndependentReferenceTests.cs:18-43).

Usage: python tests/golden/import_reference_fixtures.py [/root/reference]
"""
import base64
import hashlib
import json
import shutil
import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent


def main() -> None:
    ref = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    fx = ref / "NNtrain.Core.Tests" / "Fixtures"
    shutil.copyfile(fx / "QwenGgufReference" / "reference.gguf", HERE / "qwen_gguf_reference.gguf")
    shutil.copyfile(fx / "QwenGgufReference" / "expected.json", HERE / "qwen_gguf_expected.json")
    shutil.copyfile(fx / "IqQuantReference" / "LICENSE.llama.cpp", HERE / "LICENSE.llama.cpp")

    manifest = json.loads((HERE / "qwen_gguf_expected.json").read_text())
    digest = hashlib.sha256((HERE / "qwen_gguf_reference.gguf").read_bytes()).hexdigest()
    if digest != manifest["ggufSha256"]:
        raise SystemExit("reference.gguf does not match the sha256 in expected.json")

    src = json.loads((fx / "IqQuantReference" / "iq-quant-blocks.json").read_text())
    cases = []
    for case in src["cases"]:
        decoded = np.asarray(case["decoded"], dtype=np.float64).astype("<f4")
        if decoded.size != 256:
            raise SystemExit(f"{case['id']}: expected 256 values")
        raw = decoded.tobytes()
        if hashlib.sha256(raw).hexdigest() != case["decodedFloat32LittleEndianSha256"]:
            raise SystemExit(f"{case['id']}: float32 bits do not reproduce the recorded sha256")
        encoded = base64.b64decode(case["encoded"])
        if len(encoded) != int(case["blockBytes"]):
            raise SystemExit(f"{case['id']}: encoded size mismatch")
        cases.append({
            "id": case["id"],
            "type": int(case["type"]),
            "quantName": case["quantName"],
            "blockBytes": int(case["blockBytes"]),
            "encoded": case["encoded"],
            "decodedFloat32Base64": base64.b64encode(raw).decode("ascii"),
            "decodedFloat32LittleEndianSha256": case["decodedFloat32LittleEndianSha256"],
            "kind": case["source"].get("kind") if isinstance(case["source"], dict) else None,
        })
    out = {
        "description": "Native ggml dequantize_row_{q5_K,iq3_s,iq2_s} outputs for single 256-value blocks",
        "origin": "NNtrain.Core.Tests/Fixtures/IqQuantReference/iq-quant-blocks.json",
        "reference": src["reference"],
        "counts": src["counts"],
        "cases": cases,
    }
    (HERE / "iq_quant_blocks.json").write_text(json.dumps(out, separators=(",", ":")) + "\n")
    print(f"wrote {len(cases)} block cases, gguf sha256 ok")


if __name__ == "__main__":
    main()
