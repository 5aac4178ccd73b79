#!/usr/bin/env python3
"""Writes the committed fixtures from the CPU oracle.

The reference ships no golden vectors for this path and cannot be run, so these
fixtures freeze the oracle's output (pinned elsewhere against float64 closed
forms and autograd) on the tiny CPU-runnable configuration: they catch silent
drift of the oracle and give the GPU tests fixed bytes to compare with.

    python tests/golden/make_golden.py
"""
import hashlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from helpers import gen_scene, oracle_forward  # noqa: E402
from oracle import d3gs_oracle as O  # noqa: E402


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def main():
    O.build()
    for filt, tag in ((0, "none"), (1, "aabb"), (3, "obb")):
        scene = gen_scene(0)
        P, ref = oracle_forward(O, scene, filt)
        g, pb = O.backward(P, ref, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh,
                           scene.drgb[0], scene.dT[0])
        np.savez_compressed(
            os.path.join(HERE, f"config0_{tag}.npz"),
            radii=ref["radii"], tiles_touched=ref["tiles_touched"], workload_ranges=ref["workload_ranges"],
            gaussian_idx_sorted=ref["gaussian_idx_sorted"], n_contrib=ref["n_contrib"].astype(np.int16),
            color=ref["color"], T=ref["T"], num_rendered=np.int64(ref["num_rendered"]),
            keys_sorted_sha256=np.array(sha(ref["keys_sorted"])), scene_sha256=np.array(sha(scene.xyz) + sha(scene.color_sh)),
            dxyz=pb["dxyz"], dscale=pb["dscale"], dquat=pb["dquat"], dopacity=pb["dopacity"],
            duv=g["duv"].astype(np.float32), dconic=g["dconic"].astype(np.float32))
        print(tag, "M =", ref["num_rendered"])


if __name__ == "__main__":
    main()
