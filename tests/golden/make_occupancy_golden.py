"""Writes tests/golden/occupancy_golden.npz from the reference's own occupancy
routine, compiled from its sources where they lie (oracle/Makefile ->
oracle/_ref/libref_occupancy.so).  Runs only where /root/reference is mounted;
the .npz it writes is the committed fixture.

    python tests/golden/make_occupancy_golden.py

Contents: inputs (block, dyn_smem, static_smem, regs, dest_regs) and, per
device of DEVICES, the reference's threadBlockOccupancy for (a) 4096 seeded
random launch configurations, (b) a dense grid around every rounding boundary,
(c) out-of-range and negative inputs whose behaviour is defined in the
reference (no signed overflow).
"""
import itertools
import json
import os
import sys

import numpy as np
import yaml

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import lib as olib  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def devices():
    with open(os.path.join(ROOT, "habitat_amd", "data", "devices.yml")) as f:
        table = yaml.safe_load(f)
    v100 = dict(table["V100"])
    extra = {
        # compute capabilities the model handles differently or rejects
        "K80like_cc37": dict(v100, compute_major=3, compute_minor=7, regs_per_multiprocessor=131072,
                             shared_mem_per_multiprocessor=114688, num_sms=13),
        "M60like_cc52": dict(v100, compute_major=5, compute_minor=2, num_sms=16),
        "A100like_cc80": dict(v100, compute_major=8, compute_minor=0, num_sms=108),
        "warp48": dict(v100, warp_size=48),                       # not a power of two
        "zero_optin_smem_block0": dict(v100, shared_mem_per_block=0),
        "small_volta_pool": dict(v100, shared_mem_per_multiprocessor=20000),
    }
    table.update(extra)
    return table


def inputs():
    rng = np.random.default_rng(1234)
    n = 4096
    total = rng.integers(0, 65536, n, endpoint=True)
    stat = total // 2
    rnd = dict(block=rng.choice([32, 64, 96, 128, 192, 256, 384, 512, 768, 1024], n),
               dyn=total - stat, stat=stat, regs=rng.integers(0, 255, n, endpoint=True),
               dregs=np.where(rng.random(n) < 0.3, rng.integers(0, 255, n, endpoint=True), -1))
    blocks = [1, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, 513, 1023, 1024,
              1025, 2048]
    regs = [0, 1, 7, 8, 9, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 254, 255, 256, 257]
    smem = [0, 1, 255, 256, 257, 8191, 8192, 8193, 16384, 16385, 32768, 32769, 49151, 49152, 49153,
            65535, 65536, 65537, 98304, 163840, 163841]
    g = np.array(list(itertools.product(blocks, regs, smem)), dtype=np.int64)
    grid = dict(block=g[:, 0], dyn=g[:, 2] - g[:, 2] // 3, stat=g[:, 2] // 3, regs=g[:, 1],
                dregs=np.full(g.shape[0], -1))
    # defined-but-odd inputs: non-positive block, negative sizes (the sum wraps
    # to a small or negative int), 16-bit narrowing of the register count
    odd_rows = [
        (0, 0, 0, 32, -1), (-5, 0, 0, 32, -1), (256, -1, 0, 32, -1), (256, 0, -1, 32, -1),
        (256, -300, 0, 32, -1), (256, -600, 0, 32, -1), (256, -256, 256, 32, -1),
        (256, 1000, -1000, 32, -1), (256, 0, 0, 65535, -1), (256, 0, 0, 65536 + 32, -1),
        (256, 0, 0, 32, 65536 + 16), (256, 0, 0, 32, 300), (256, 0, 0, 300, 20),
        (1 << 20, 0, 0, 16, -1), (256, 1 << 30, 0, 16, -1), (256, 1 << 30, 1 << 30, 16, -1),
        (256, -(1 << 31), 0, 16, -1), (256, (1 << 31) - 1, -(1 << 31) + 1, 16, -1),
        (1024, 49152, 0, 64, -1), (1024, 0, 49152, 64, -1), (64, 24576, 24577, 16, -1),
    ]
    o = np.array(odd_rows, dtype=np.int64)
    odd = dict(block=o[:, 0], dyn=o[:, 1], stat=o[:, 2], regs=o[:, 3], dregs=o[:, 4])
    cat = {k: np.concatenate([rnd[k], grid[k], odd[k]]).astype(np.int64) for k in rnd}
    # keep only rows the reference evaluates without signed overflow:
    # (int)(static + dyn) + 255 must fit an int
    tot = ((cat["stat"] + cat["dyn"] + 2**31) % 2**32) - 2**31
    keep = tot <= 2**31 - 1 - 255
    return {k: v[keep].astype(np.int32) for k, v in cat.items()}


def main():
    ref = olib.ref()
    if ref is None:
        raise SystemExit("the reference tree is not mounted: cannot regenerate the fixture")
    inp = inputs()
    devs = devices()
    out = dict(inp)
    names = []
    for name, props in devs.items():
        d = olib.make_device(**props)
        occ_own = olib.ref_occupancy_batch(d, inp["block"], inp["dyn"], inp["stat"], inp["regs"])
        occ_lut = olib.ref_occupancy_batch(d, inp["block"], inp["dyn"], inp["stat"], inp["regs"],
                                           inp["dregs"])
        out["occ_own__" + name] = occ_own.astype(np.int32)
        out["occ_lut__" + name] = occ_lut.astype(np.int32)
        names.append(name)
    np.savez_compressed(os.path.join(HERE, "occupancy_golden.npz"), **out)
    with open(os.path.join(HERE, "occupancy_golden_devices.json"), "w") as f:
        json.dump({n: devs[n] for n in names}, f, indent=1, sort_keys=True)
    print("rows", inp["block"].shape[0], "devices", len(names))


if __name__ == "__main__":
    main()
