#!/usr/bin/env python3
"""Writes tests/golden/codec_vectors.bin and codec_vectors.json: the contract of compression_8bit /
decompression_8bit (source/clusterKernels.cu:1135-1232) frozen as data.

Inputs: the table's 126 values with both fp32 neighbours, the 125 midpoints of adjacent entries with two
patterns either side, both thresholds (1.5e-6, 0.995703), 1.0 and the last entry with four patterns either
side, zeros, denormals, round numbers, the sliver 0.99140614 < a <= 0.995703, overflow; all of it with both
signs.  For every precision p of PRECISIONS the scaled inputs are xs = fl32(x * fl32(p)) and the file holds the
codes of xs under p for both readings of the one place where the reference reads a table slot it never wrote
(sliver rule 0: the slot holds 1.0, codes 125 / 253; rule 1: the slot holds 0.0, codes 126 / 254), and the
256-entry decode table.  Produced by the CPU checker (oracle/), whose two formulations must agree on every
vector before anything is written.  CPU only.

Layout of the .bin (little endian), in order:
  x            N float32
  then per precision, in the order of the .json: codes_rule0 N uint8, codes_rule1 N uint8, decode_lut 256 float32
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402

PRECISIONS = [1.0, 0.1, 3.7, 2.0 ** -40, -1.0]


def inputs():
    t = oracle.table()
    pts = [t, np.nextafter(t, np.float32(0)), np.nextafter(t, np.float32(2))]
    mids = ((t[:-1].astype(np.float64) + t[1:].astype(np.float64)) / 2).astype(np.float32)
    for k in (-2, -1, 0, 1, 2):
        pts.append((mids.view(np.uint32).astype(np.int64) + k).astype(np.uint32).view(np.float32))
    for thr in (np.float32(0.0000015), np.float32(0.995703), np.float32(1.0), t[125]):
        b = int(np.array([thr]).view(np.uint32)[0])
        pts.append(np.arange(b - 4, b + 5, dtype=np.uint32).view(np.float32))
    pts.append(np.array([0.0, 1e-45, 1e-38, 1.1754944e-38, 0.5, 0.25, 0.1, 0.01, 0.001, 0.992, 0.993, 0.994,
                         0.995, 0.9957, 0.9958, 1.0, 1.5, 3e38], np.float32))
    x = np.concatenate([np.asarray(p, np.float32).reshape(-1) for p in pts])
    return np.concatenate([x, -x]).astype("<f4")


def main():
    x = inputs()
    blobs = [x.tobytes()]
    meta = {"n": int(x.size), "dtype_x": "<f4", "scaling": "xs = float32(x * float32(precision))",
            "sliver": "0.99140614 < |xs / precision| <= 0.995703: rule 0 gives 125 / 253, rule 1 gives 126 / 254",
            "reference": "source/clusterKernels.cu:1135-1232", "precisions": []}
    for p in PRECISIONS:
        with np.errstate(all="ignore"):
            xs = (x * np.float32(p)).astype(np.float32)
        per = {"precision": float(np.float32(p)), "precision_bits": "0x%08x" % int(np.array([p], "<f4").view(np.uint32)[0])}
        for rule in (0, 1):
            a = oracle.compress(xs, p, rule, "literal")
            b = oracle.compress(xs, p, rule, "closed")
            if not np.array_equal(a, b):
                raise SystemExit("the checker's two formulations disagree at precision %r, rule %d" % (p, rule))
            blobs.append(a.astype(np.uint8).tobytes())
            per["differs_from_rule0" if rule else "codes_sha256"] = (
                int((a != oracle.compress(xs, p, 0, "literal")).sum()) if rule else hashlib.sha256(a.tobytes()).hexdigest())
        blobs.append(oracle.decode_lut(p).astype("<f4").tobytes())
        meta["precisions"].append(per)
    raw = b"".join(blobs)
    meta["bytes"] = len(raw)
    meta["sha256"] = hashlib.sha256(raw).hexdigest()
    open(os.path.join(HERE, "codec_vectors.bin"), "wb").write(raw)
    with open(os.path.join(HERE, "codec_vectors.json"), "w") as f:
        json.dump(meta, f, indent=1)
        f.write("\n")
    print("wrote %d inputs x %d precisions, %d bytes" % (x.size, len(PRECISIONS), len(raw)))


if __name__ == "__main__":
    main()
