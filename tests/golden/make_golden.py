"""Extracts golden vectors that the reference's own tests hold into small JSON fixtures.

Run once in a container that mounts the reference tree (default /root/reference):

    python tests/golden/make_golden.py [/path/to/reference]

It only READS data tables as text; it imports and executes nothing from the reference.
Outputs (committed next to this script):
  mxfp4_llamacpp_dequant.json  -- external/ds4-dump/quants_selftest_expected.inc
      `expected_mxfp4[256]`: f32 bit patterns produced by llama.cpp's
      dequantize_row_mxfp4 for the 8 blocks that quants_selftest.c:82-87,102-105 builds
      (LCG s = s*1664525 + 1013904223, byte = s >> 24, seed 0x3333 over 8*17 bytes, then
      the scale byte of block i forced to 120 + i).
"""
import json
import os
import re
import sys


def parse_u32_table(text: str, name: str):
    m = re.search(r"%s\[(\d+)\]\s*=\s*\{(.*?)\};" % re.escape(name), text, re.S)
    if not m:
        raise SystemExit(f"table {name} not found")
    vals = [int(v, 16) for v in re.findall(r"0x[0-9a-fA-F]+", m.group(2))]
    assert len(vals) == int(m.group(1)), (len(vals), m.group(1))
    return vals


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    here = os.path.dirname(os.path.abspath(__file__))
    inc = open(os.path.join(ref, "external/ds4-dump/quants_selftest_expected.inc")).read()
    out = {
        "source": "external/ds4-dump/quants_selftest_expected.inc (expected_mxfp4)",
        "construction": {"lcg_mul": 1664525, "lcg_add": 1013904223, "seed": 0x3333,
                         "n_blocks": 8, "block_bytes": 17, "e_base": 120},
        "f32_bits": parse_u32_table(inc, "expected_mxfp4"),
    }
    with open(os.path.join(here, "mxfp4_llamacpp_dequant.json"), "w") as f:
        json.dump(out, f)
    print("wrote mxfp4_llamacpp_dequant.json", len(out["f32_bits"]))


if __name__ == "__main__":
    main()
