#!/usr/bin/env python3
"""Turns the CSV of stream_sweep into the text table kept under profiles/: python3 summarize.py sweep.csv > table.txt"""
import collections
import csv
import sys

NAMES = {0: "R4    read fp32", 1: "R4W1  read fp32, write 1 byte each (compression's pattern)",
         2: "R1W4  read bytes, write fp32 (decompression's pattern)", 3: "R4W4  copy fp32", 4: "W4    write fp32",
         5: "R4W1W as R4W1 with 16-byte stores of the bytes", 6: "R1W4W as R1W4 with 16-byte loads of the bytes"}
POLICY = {0: "plain", 1: "sc0", 2: "nt", 16: "sc1", 17: "sc0 sc1", 19: "sc0 sc1 nt"}
N = 819200000
PEAK = 8000.0


def mapping(r):
    if r["waves_per_cu"] == 0:
        return "a workgroup per tile"
    if r["xcd_remap"] == 2:
        return "tiles drawn from a counter"
    if r["chunk_tiles"] == 1:
        return "grid-stride"
    tiles = N // (r["T"] * r["U"] * 4)
    whole = r["chunk_tiles"] == (tiles + r["grid"] - 1) // r["grid"]
    return ("one range per workgroup" if whole else "2 MiB chunks") + (", XCD-adjacent" if r["xcd_remap"] else "")


def main():
    rows, outside = [], []
    for r in csv.DictReader(open(sys.argv[1])):
        if not r["kind"].isdigit():
            outside.append(r)
            continue
        for k in ("kind", "load_policy", "store_policy", "U", "T", "chunk_tiles", "xcd_remap", "wait_for_stores", "waves_per_cu", "grid"):
            r[k] = int(r[k])
        r["g"] = float(r["GBps_med"])
        r["map"] = mapping(r)
        rows.append(r)
    print("GB/s are medians of the timed launches (algorithmic bytes of the pattern / duration); % of the 8 TB/s HBM peak in brackets.")
    print("%d measurements of %d kernels.\n" % (len(rows), len({(r['kind'], r['load_policy'], r['store_policy'], r['U'], r['T']) for r in rows})))
    print("The HIP runtime's own movers on the same buffers:")
    for r in outside:
        print("  %-14s %7.0f GB/s (%.1f %%)" % (r["kind"], float(r["GBps_med"]), 100 * float(r["GBps_med"]) / PEAK))
    print()
    for kind in sorted(NAMES):
        kr = sorted((r for r in rows if r["kind"] == kind), key=lambda r: -r["g"])
        if not kr:
            continue
        print("== %s: best %0.f GB/s (%.1f %%)" % (NAMES[kind], kr[0]["g"], 100 * kr[0]["g"] / PEAK))
        print("   the eight fastest settings:")
        for r in kr[:8]:
            print("   %7.0f  loads %-10s stores %-10s %2d x 16 B per lane, %4d lanes, %2d waves/CU, %s%s" % (
                r["g"], POLICY[r["load_policy"]], POLICY[r["store_policy"]], r["U"], r["T"], r["waves_per_cu"], r["map"],
                ", waits for its stores" if r["wait_for_stores"] else ""))
        for key, label in (("store_policy", "store policy"), ("load_policy", "load policy"), ("U", "16-byte vectors per lane and tile"),
                           ("T", "lanes per workgroup"), ("map", "mapping"), ("waves_per_cu", "wavefronts per CU"),
                           ("wait_for_stores", "waits for its stores")):
            best = collections.OrderedDict()
            for r in sorted(kr, key=lambda r: str(r[key]) if key == "map" else r[key]):
                best[r[key]] = max(best.get(r[key], 0.0), r["g"])
            if len(best) > 1:
                print("   best by %s: %s" % (label, ", ".join("%s %.0f" % (POLICY.get(k, k) if "policy" in key else k, g) for k, g in best.items())))
        print()


if __name__ == "__main__":
    main()
