"""Per-workgroup timeline of one launch of the forward kernel for short lists.

The kernel carries time stamps (10 ns real-time counter) that are compiled in only with ``-DHSTU_TIMELINE``: at entry,
when its offsets are in, at the first step of the key sweep, at the end of the sweep and at exit.  This example builds
such a variant of the library next to the shipped one (``--build``, on a machine with hipcc; about two minutes),
runs one launch of a named configuration on it and prints the phases as min / median / max over the workgroups, per
level (level 0 = the highest, heaviest query tile) and per XCD.

    python ops-rec_amd/examples/hstu_fwd_timeline.py --build          # here, where hipcc is
    python ops-rec_amd/examples/hstu_fwd_timeline.py [--workload C2]  # on the GPU box
"""

from __future__ import annotations

import argparse
import os
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(_HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(_HERE)))

from ops_rec import _build  # noqa: E402

TIMELINE_LIB = os.path.join(_build.LIB_DIR, "timeline", "libhstu_mi355.so")


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--build", action="store_true", help="compile the library with -DHSTU_TIMELINE and exit")
    ap.add_argument("--workload", default="C2")
    ap.add_argument("--burst", type=int, default=1, help="launches back to back; the stamps are those of the last one")
    ap.add_argument("--shape", default=None, help="batch,heads,shortest,longest at head dim 128 instead of a named workload")
    args = ap.parse_args()
    if args.build:
        print(_build.build(verbose=False, extra_flags=("-DHSTU_TIMELINE",), lib_path=TIMELINE_LIB))
        return
    if not os.path.exists(TIMELINE_LIB):
        raise SystemExit(f"{TIMELINE_LIB} is missing: run this example with --build first")
    _build.LIB_PATH = TIMELINE_LIB  # before the library is loaded
    import numpy as np
    import torch

    from ops_rec import _native, _ops, workloads

    dev = "cuda:0"
    if args.shape:
        batch, heads, lo, hi = (int(v) for v in args.shape.split(","))
        w = workloads.make("shape", dtype=torch.bfloat16, device=dev, dim=128, batch=batch, heads=heads, lo=lo, hi=hi)
        args.workload = args.shape
    else:
        w = workloads.config(args.workload).to(dev)
    buf = torch.zeros(1 << 20, dtype=torch.int64, device=dev)  # 8 words per workgroup
    os.environ["HSTU_TIMELINE_BUFFER"] = str(buf.data_ptr())
    os.environ["HSTU_MI355_SHORT"] = "1"
    _native.reload_switches()
    p = _ops.prepare_forward(w.q, w.k, w.v, None, None, w.mask_type, w.max_seq_len, w.max_seq_len, w.silu_scale,
                             w.seq_offset, w.seq_offset, w.num_context, w.num_target, w.target_group_size, w.alpha)  # fmt: skip
    if not p.kernel_name().endswith("_short"):
        raise SystemExit(f"{args.workload} is not taken by the kernel for short lists ({p.kernel_name()})")
    for _ in range(5):
        p.launch()
    torch.cuda.synchronize()
    buf.zero_()
    torch.cuda.synchronize()
    for _ in range(args.burst):  # (every launch overwrites the records: what is read back is the last one)
        p.launch()
    torch.cuda.synchronize()
    r = buf.cpu().numpy().reshape(-1, 8)
    r = r[r[:, 0] != 0]
    t0 = r[:, 0].min()

    def us(x):
        return (x - t0) / 100.0

    def stats(x):
        return f"min {x.min():6.2f}  median {np.median(x):6.2f}  max {x.max():6.2f}"

    live = r[:, 6] == 1
    dead, lv = r[~live], r[live]
    print(f"{args.workload}: {p.kernel_name()}, {len(r)} workgroups, {int(live.sum())} with a query tile, "
          f"launch span {us(r[:, 4].max()):.2f} us (all times in us)")
    if len(dead):
        print(f"workgroups without a tile: entry {stats(us(dead[:, 0]))}; lifetime {stats((dead[:, 4] - dead[:, 0]) / 100.0)}")
    print("entry                      ", stats(us(lv[:, 0])))
    print("entry -> offsets in        ", stats((lv[:, 1] - lv[:, 0]) / 100.0))
    print("offsets in -> first step   ", stats((lv[:, 2] - lv[:, 1]) / 100.0))
    print("key sweep                  ", stats((lv[:, 3] - lv[:, 2]) / 100.0))
    print("rows stored, exit          ", stats((lv[:, 4] - lv[:, 3]) / 100.0))
    print("exit                       ", stats(us(lv[:, 4])))
    level = lv[:, 7] & 0xFFFF
    for lvl in sorted(set(level.tolist())):
        m = level == lvl
        sweep = (lv[m, 3] - lv[m, 2]) / 100.0
        print(f"level {lvl:2d}: {int(m.sum()):4d} tiles | entry median {np.median(us(lv[m, 0])):6.2f} max {us(lv[m, 0]).max():6.2f}"
              f" | sweep median {np.median(sweep):6.2f} max {sweep.max():6.2f} | exit median {np.median(us(lv[m, 4])):6.2f}"
              f" max {us(lv[m, 4]).max():6.2f}")
    xcc = (lv[:, 5] >> 32) & 0xF
    for x in range(8):
        m = xcc == x
        if m.any():
            print(f"XCD {x}: {int(m.sum()):4d} tiles | last exit {us(lv[m, 4]).max():6.2f} | resident time summed "
                  f"{((lv[m, 4] - lv[m, 0]) / 100.0).sum():8.1f}")
    ts = np.arange(0, us(r[:, 4].max()), 2.0)
    print("workgroups with a tile resident, every 2 us:",
          [int(((us(lv[:, 0]) <= t) & (us(lv[:, 4]) > t)).sum()) for t in ts])


if __name__ == "__main__":
    main()
