"""Writes the fixtures under tests/golden/.  Run from the repo root:

    python tests/golden/make_fixtures.py

* best_known_labels.json -- the label strings and p50 TFLOP/s of the reference's
  perf-regression registry (a data file its own tests hold:
  contrib/kittens/test/bench/tools/best_known.json), read as JSON.
* kat.json -- known-answer cases transcribed from the reference's instruction
  tests (operand bytes, scales, expected value) with the file:line of each.

Nothing of the reference is imported or executed.
"""

import json
import os

HERE = os.path.dirname(os.path.abspath(__file__))
REF = "/root/reference"


def labels():
    with open(os.path.join(REF, "contrib/kittens/test/bench/tools/best_known.json")) as f:
        bk = json.load(f)
    out = []
    for mcpu, benches in bk.items():
        for bench, sizes in benches.items():
            for size, entries in sizes.items():
                for e in entries:
                    out.append({"mcpu": mcpu, "bench": bench, "size": size, "label": e["label"],
                                "expected_tflops": e["expected_tflops"]})
    return out


KAT = {
    "comment": "closed-form known answers held by the reference's instruction tests",
    "cases": [
        {"name": "bf16_16x16x32_all_ones", "source": "test/integration/test_mfma_cdna4_doubled_k_e2e.py:77-134",
         "dtype": "bf16", "a_bits": "0x3F80", "b_bits": "0x3F80", "k": 32, "expected": 32.0},
        {"name": "bf16_32x32x16_all_ones", "source": "test/integration/test_mfma_cdna4_doubled_k_e2e.py:77-134",
         "dtype": "bf16", "a_bits": "0x3F80", "b_bits": "0x3F80", "k": 16, "expected": 16.0},
        {"name": "fp8_scaled_nonidentity", "source": "test/integration/test_mfma_f8f6f4_e2e.py:39-66",
         "dtype": "fp8_e4m3", "a_byte": "0x3E", "b_byte": "0x3A", "a_value": 1.75, "b_value": 1.25,
         "scale_a_e8m0": "0x81", "scale_b_e8m0": "0x80", "scale_a": 4.0, "scale_b": 2.0, "k": 128,
         "expected": 2240.0},
        {"name": "fp8_split_k_accum", "source": "test/integration/test_mfma_f8f6f4_e2e.py:68-95",
         "dtype": "fp8_e4m3", "a_bytes_halves": ["0x38", "0x3C"], "b_bytes_halves": ["0x40", "0x30"],
         "a_values_halves": [1.0, 1.5], "b_values_halves": [2.0, 0.5], "scale_e8m0": "0x7F",
         "c_init": 10.0, "k": 128, "expected": 186.0},
    ],
    "e4m3_codes": {"0x38": 1.0, "0x3C": 1.5, "0x3E": 1.75, "0x3A": 1.25, "0x40": 2.0, "0x30": 0.5,
                   "0x7E": 448.0},
    "e8m0_codes": {"0x7F": 1.0, "0x80": 2.0, "0x81": 4.0},
    "estimator_anchors": [
        {"label": "m4096xn4096xk4096_wg32x16x1_w1x4x1_twg8x16x1_pipestrat11_wgcu1_lcm1_um1_epeel1_llsched1_hoistwait1_rotc1_lt_flat_cdna4",
         "operand_path": "direct_b", "vgprs": 234, "agprs": 128, "lds": 32768, "simd_occupancy": 1},
        {"label": "m2048xn4096xk4096_wg16x32x1_w1x4x1_twg8x8x2_pipestrat3_wgcu1_lcm1_um3_epeel1_llsched1_hoistwait0_rotc1_lt_flat_cdna4",
         "operand_path": "direct_b", "vgprs": 154, "agprs": 64, "lds": 49152},
    ],
}


def main():
    with open(os.path.join(HERE, "best_known_labels.json"), "w") as f:
        json.dump(labels(), f, indent=1)
    with open(os.path.join(HERE, "kat.json"), "w") as f:
        json.dump(KAT, f, indent=1)


if __name__ == "__main__":
    main()
