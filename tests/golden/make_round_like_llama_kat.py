"""Writes round_like_llama_kat.json: the inputs and expected outputs the
reference's own tests of its activation rounding hold
(src/ref/matmul.zig:382-419), as bit patterns. Nothing of the reference is run:
the vectors are typed from its tests' literals, and the one expected value the
reference computes (`d`, an f16 rounding of amax / 127) is evaluated with
numpy's float16 here.

    python tests/golden/make_round_like_llama_kat.py
"""
import json
import os

import numpy as np


def bits(a):
    return [int(v) for v in np.asarray(a, dtype=np.float32).view(np.uint32)]


def main():
    cases = []
    # 'Q8_K and actual x86 Q8_0 round halfway values to even' (matmul.zig:394-406)
    x = np.zeros(256, dtype=np.float32)
    x[0] = 127
    x[1:7] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5]
    x[7] = -0.1
    # The reference compares these six as floats (a zero of either sign passes:
    # under Q8_K the scale is -1 here) and the eighth Q8_0 value as bits.
    halves = bits(np.float32([0, 2, 2, 0, -2, -2]))
    cases.append({"name": "ties_to_even_q8_k", "type": "q4_k", "input": bits(x),
                  "expect": {"first": 1, "bits": halves, "compare": "value"}})
    cases.append({"name": "ties_to_even_x86_q8_0", "type": "q8_0", "input": bits(x),
                  "expect": {"first": 1, "bits": halves + [0], "compare": "bits"}})
    # 'actual x86 Q8_0 uses 127 over amax before rounding' (matmul.zig:408-419)
    x = np.zeros(32, dtype=np.float32)
    x.view(np.uint32)[0] = 0x3F80000F
    x.view(np.uint32)[1] = 0x3CA14298
    x[2] = -x[1]
    d = np.float32(np.float16(x[0] / np.float32(127)))
    cases.append({"name": "127_over_amax_before_rounding", "type": "q8_0", "input": bits(x),
                  "expect": {"first": 0, "bits": bits([np.float32(127) * d, np.float32(2) * d, np.float32(-2) * d]), "compare": "bits"}})
    # 'IQ4_XS llama.cpp activations use Q8_K rounding' (matmul.zig:382-392):
    # the rounding changes the row, and IQ4_XS rounds exactly as Q6_K does.
    x = ((np.arange(512) % 41).astype(np.float32) - np.float32(20)) / np.float32(23)
    x[0] = 2.75
    x[256] = -3.25
    cases.append({"name": "iq4_xs_rounds_like_q8_k", "type": "iq4_xs", "same_as_type": "q6_k", "input": bits(x)})
    out = {"source": "reference src/ref/matmul.zig:382-419 (tests of roundLikeLlama); values are f32 bit patterns", "cases": cases}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "round_like_llama_kat.json")
    with open(path, "w") as f:
        json.dump(out, f)
        f.write("\n")


if __name__ == "__main__":
    main()
