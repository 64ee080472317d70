#!/usr/bin/env python3
"""Writes the golden fixtures of this directory from the CPU oracle.

    python tests/golden/make_fixtures.py

bundle_header_v1.json   tensor list + alignment -> header bytes (hex), by the
                        oracle's independent struct-based codec
small_bundle_v1.json    seeded byte chunks -> packed payload (hex) for the tight
                        (align 1) and the 256-byte aligned layout
argument_structure_v1.json  nested argument lists (tensors named by letters) -> flat
                        tensor order, group sizes and the framing bytes (hex)
kat_patterns.json       the closed-form patterns of the reference's own tests
                        (segment lengths and fill rule; expected = the running
                        pattern), so the data the reference tests hold is kept
                        as data next to the tests that use it

The header format is this build's own (the reference serialises its header with
cista, whose byte layout has no fixture in the reference), so these vectors pin
stability of the format, not parity with the reference.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402


def main():
    tensors = [
        {"device": [10, 0], "dtype": [2, 32, 1], "shape": [16384]},
        {"device": [10, 0], "dtype": [4, 16, 1], "shape": [3, 5, 7]},
        {"device": [10, 0], "dtype": [0, 8, 1], "shape": [301]},
        {"device": [1, 0], "dtype": [2, 16, 1], "shape": []},
        {"device": [10, 1], "dtype": [0, 32, 1], "shape": [0, 9]},
        {"device": [11, 0], "dtype": [1, 64, 2], "shape": [2, 2]},
    ]
    cases = []
    for align in (1, 16, 256, 4096):
        blob = oracle.encode_header([{"device": tuple(t["device"]), "dtype": tuple(t["dtype"]),
                                      "shape": tuple(t["shape"])} for t in tensors], align)
        cases.append({"align": align, "header_hex": blob.hex()})
    with open(os.path.join(HERE, "bundle_header_v1.json"), "w") as f:
        json.dump({"tensors": tensors, "cases": cases}, f, indent=1)

    rng = np.random.default_rng(20240521)
    sizes = [0, 1, 15, 16, 17, 255, 256, 257, 1000, 4099]
    chunks = [rng.integers(0, 256, size=n, dtype=np.uint8) for n in sizes]
    small = {"chunks_hex": [c.tobytes().hex() for c in chunks], "packed": {}}
    for align in (1, 256):
        small["packed"][str(align)] = oracle.pack(chunks, align).tobytes().hex()
    with open(os.path.join(HERE, "small_bundle_v1.json"), "w") as f:
        json.dump(small, f, indent=1)

    # the reference's own example first (bindings_runtime_helpers.hpp:364-386)
    arg_cases = [
        [[["a", "b"], ["c"]]],
        ["a", ["b", "c"], [["d"], [], ["e", "f"]], ["g"], [], "h"],
        [[[], [], ["a"]], [["b", "c", "d"]]],
        [],
    ]
    out = []
    for args in arg_cases:
        flat, structure = oracle.flatten_arguments(args, lambda x: isinstance(x, str))
        out.append({"args": args, "flat": flat, "structure": [[k, c] for k, c in structure],
                    "blob_hex": oracle.encode_argument_structure(structure).hex()})
    with open(os.path.join(HERE, "argument_structure_v1.json"), "w") as f:
        json.dump(out, f, indent=1)

    kat = {
        "fill_rule": "byte k of the concatenated stream = k mod 256",
        "iov_small": [256, 512, 300],
        "iov_large": [512 * 1024, 256 * 1024, 800 * 1024],
        "split": {"buffer_bytes": 100, "sizes": [10, 20, 30, 40], "offsets": [0, 10, 30, 60]},
        "split_overflow": {"buffer_bytes": 100, "sizes": [50, 51]},
        "float_iov": {"segments": 4, "bytes_per_segment": 8192, "value_rule": "float(i mod 256), i global"},
        "process": {"value_rule": "float(i mod 256)", "expected_rule": "float(i mod 256) / 2"},
    }
    with open(os.path.join(HERE, "kat_patterns.json"), "w") as f:
        json.dump(kat, f, indent=1)


if __name__ == "__main__":
    main()
