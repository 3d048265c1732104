"""Writes tests/golden/sched_fixtures.json from the reference's own scheduler
headers compiled in place (oracle/_ref/libcatcoc_ref_sched.so, built by
oracle/Makefile from /root/reference).  Run in the authoring container only:

    python tests/golden/make_sched_fixtures.py

The JSON holds data only: task index -> tile coordinates / edge shapes.
"""
import ctypes as C
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402

u32 = C.c_uint32


def main():
    oracle.build()
    ref = oracle.ref_sched()
    if ref is None:
        raise SystemExit("oracle/_ref/libcatcoc_ref_sched.so not built (reference tree absent?)")
    fx = {"swizzle": [], "splitk": [], "allgather": []}

    # (off, dir, M, N, m0, n0): the five benchmark configs' grids plus ragged ones
    base_cases = [
        (7, 1, 1024, 4096, 128, 256),   # W8A8 reduce-scatter sub-problem (8192/8 rows)
        (7, 1, 512, 4096, 128, 256),    # fp16 reduce-scatter sub-problem (4096/8 rows)
        (7, 1, 512, 1024, 128, 256),    # all-reduce, fp16
        (7, 1, 2, 8192, 128, 256),      # decode M=16, P=8
        (7, 1, 1000, 1696, 128, 256),   # ragged both ways
        (7, 0, 2048, 1000, 128, 256),
        (3, 0, 1300, 700, 128, 256),
        (3, 1, 1300, 2100, 128, 256),
        (1, 0, 384, 512, 128, 256),
        (2, 1, 640, 1280, 128, 256),
        (4, 0, 128, 256, 128, 256),     # single tile
    ]
    for off, d, M, N, m0, n0 in base_cases:
        o = (u32 * 5)()
        assert ref.ref_swizzle_coord(u32(off), u32(d), u32(M), u32(N), u32(m0), u32(n0), u32(0), o)
        loops = o[4]
        rows = []
        for t in range(loops):
            ref.ref_swizzle_coord(u32(off), u32(d), u32(M), u32(N), u32(m0), u32(n0), u32(t), o)
            rows.append([o[0], o[1], o[2], o[3]])
        fx["swizzle"].append({"off": off, "dir": d, "M": M, "N": N, "m0": m0, "n0": n0, "coords": rows})

    split_cases = [
        (7, 1, 16, 8192, 8192, 128, 256, 256, 8),
        (3, 0, 512, 8192, 8192, 128, 256, 256, 2),
        (3, 0, 100, 700, 1800, 128, 256, 256, 3),
        (1, 1, 128, 512, 2304, 128, 256, 256, 4),
        (7, 1, 64, 1024, 1000, 64, 256, 128, 5),
    ]
    for off, d, M, N, K, m0, n0, k0, f in split_cases:
        o = (u32 * 8)()
        assert ref.ref_splitk_coord(u32(off), u32(d), u32(M), u32(N), u32(K), u32(m0), u32(n0), u32(k0), u32(f), u32(0), o)
        loops = o[7]
        rows = []
        for t in range(loops):
            ref.ref_splitk_coord(u32(off), u32(d), u32(M), u32(N), u32(K), u32(m0), u32(n0), u32(k0), u32(f), u32(t), o)
            rows.append([o[i] for i in range(7)])
        fx["splitk"].append({"off": off, "dir": d, "M": M, "N": N, "K": K, "m0": m0, "n0": n0, "k0": k0, "f": f,
                             "coords": rows})

    ag_cases = [
        (7, 1, 8, 1, 512, 1024, 128, 256),   # all-gather benchmark config, commInterval 1 (example default)
        (7, 1, 8, 3, 512, 1024, 128, 256),   # ragged last round (4 tile rows per rank, 3 per round)
        (7, 1, 2, 2, 768, 640, 128, 256),
        (3, 0, 4, 2, 640, 1000, 128, 256),
    ]
    for off, d, P, ci, ml, N, m0, n0 in ag_cases:
        o = (u32 * 5)()
        assert ref.ref_allgather_coord(u32(off), u32(d), u32(P), u32(ci), u32(ml), u32(N), u32(m0), u32(n0), u32(0), o)
        loops = o[4]
        rows = []
        for t in range(loops):
            ref.ref_allgather_coord(u32(off), u32(d), u32(P), u32(ci), u32(ml), u32(N), u32(m0), u32(n0), u32(t), o)
            rows.append([o[0], o[1], o[2], o[3]])
        fx["allgather"].append({"off": off, "dir": d, "P": P, "commInterval": ci, "mLocal": ml, "N": N,
                                "m0": m0, "n0": n0, "coords": rows})

    with open(os.path.join(HERE, "sched_fixtures.json"), "w") as f:
        json.dump(fx, f, separators=(",", ":"))
    print("wrote", sum(len(c["coords"]) for k in fx for c in fx[k]), "coords")


if __name__ == "__main__":
    main()
