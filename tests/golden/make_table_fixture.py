"""Writes tests/golden/8bit_floats_table.bin: the raw payload of the reference's codebook file.

The reference keeps its 126-entry table in source/8bit_floats.hdf5 (dataset /Default, 126x1 fp32,
contiguous layout, little-endian payload at byte offset 2144, file length 2648).  No HDF5 library
exists in this image, so the payload is cut out by offset; the superblock signature and the file
length are checked first.  Run only where the reference tree is mounted.
"""
import hashlib
import os
import sys

SRC = "/root/reference/source/8bit_floats.hdf5"
DST = os.path.join(os.path.dirname(os.path.abspath(__file__)), "8bit_floats_table.bin")


def main():
    raw = open(SRC, "rb").read()
    assert raw[:8] == b"\x89HDF\r\n\x1a\n", "not an HDF5 file"
    assert len(raw) == 2648, len(raw)
    payload = raw[2144:2648]
    open(DST, "wb").write(payload)
    print(DST, len(payload), hashlib.sha256(payload).hexdigest())


if __name__ == "__main__":
    sys.exit(main())
