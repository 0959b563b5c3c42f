"""How much of the offload / prefetch copies ran beside the kernels of a training step.

Works on intervals (kind, start, stop): `compute` for kernels, `d2h` / `h2d` for the copies over the host link.
    copy busy      = length of the union of the copies' intervals
    compute busy   = length of the union of the kernels' intervals
    overlap        = length of (union of copies) intersected with (union of kernels)
    overlap fraction = overlap / copy busy: the share of the link's time that was hidden behind compute
    duplex         = length of (union of d2h) intersected with (union of h2d): both directions of the link at once

Two sources give the intervals: the library's own per-launch HIP events (vdnn_profile_intervals; bench.py uses
`from_profile`), and a rocprofv3 trace of the same program, which this module reads when run as a script:

    rocprofv3 --kernel-trace --memory-copy-trace --output-format csv -d DIR -- python3 bench.py ...
    python3 -m vdnn_implementation_amd.trace_overlap DIR

From a trace, only what lies between the first and the last matrix-core kernel is counted, so the uploads of
parameters and inputs before the first step and the downloads after the last are left out.
"""
import csv
import glob
import os
import sys

LINK_COPY_CLASSES = ("offload_d2h", "offload_zvc_copy", "offload_zvc", "prefetch_h2d", "prefetch_zvc")


def union(intervals):
    """Sorted, disjoint intervals covering the same points as `intervals`."""
    out = []
    for a, b in sorted(intervals):
        if b <= a:
            continue
        if out and a <= out[-1][1]:
            out[-1][1] = max(out[-1][1], b)
        else:
            out.append([a, b])
    return out


def length(u):
    return sum(b - a for a, b in u)


def intersect(u, v):
    """Intersection of two sorted disjoint interval lists."""
    out, i, j = [], 0, 0
    while i < len(u) and j < len(v):
        a, b = max(u[i][0], v[j][0]), min(u[i][1], v[j][1])
        if a < b:
            out.append([a, b])
        if u[i][1] < v[j][1]:
            i += 1
        else:
            j += 1
    return out


def summarize(intervals):
    """intervals: iterable of (kind, start, stop), kind in {"compute", "d2h", "h2d"}; times in one unit (returned as is)."""
    by = {"compute": [], "d2h": [], "h2d": []}
    for kind, a, b in intervals:
        by[kind].append((a, b))
    compute, d2h, h2d = union(by["compute"]), union(by["d2h"]), union(by["h2d"])
    copies = union(by["d2h"] + by["h2d"])
    busy = length(copies)
    everything = union(by["compute"] + by["d2h"] + by["h2d"])
    span = (everything[-1][1] - everything[0][0]) if everything else 0.0
    hidden = length(intersect(copies, compute))
    return {"span": span, "compute_busy": length(compute), "copy_busy": busy, "d2h_busy": length(d2h), "h2d_busy": length(h2d),
            "copy_beside_compute": hidden, "overlap_fraction": hidden / busy if busy else None,
            "duplex": length(intersect(d2h, h2d)), "copy_exposed": busy - hidden}


def from_profile(records):
    """records: (class name, stream, start ms, stop ms) as vdnn_profile_intervals returns them. Kernels of the compute
    stream count as compute; the copy engine's transfers and the kernels that read or write pinned host memory count as
    copies. The kernel that packs a tensor on the packing stream is neither: it works at HBM speed beside the layer's
    own kernels and is what the compressed offload costs, not what it moves."""
    out = []
    for name, stream, a, b in records:
        if name in LINK_COPY_CLASSES:
            out.append(("d2h" if name.startswith("offload") else "h2d", a, b))
        elif stream == 0:
            out.append(("compute", a, b))
    return out


def _read(path):
    with open(path, newline="") as f:
        return list(csv.DictReader(f))


def from_rocprof(directory):
    """Intervals (ns) from the kernel_trace / memory_copy_trace CSV files under `directory` (searched recursively)."""
    kernels, copies = [], []
    for path in glob.glob(os.path.join(directory, "**", "*kernel_trace.csv"), recursive=True):
        kernels += _read(path)
    for path in glob.glob(os.path.join(directory, "**", "*memory_copy_trace.csv"), recursive=True):
        copies += _read(path)
    if not kernels:
        raise SystemExit("no *kernel_trace.csv under %s" % directory)
    mfma = [k for k in kernels if "igemm" in k["Kernel_Name"]]
    if not mfma:
        raise SystemExit("no matrix-core kernel in the trace")
    t0 = min(int(k["Start_Timestamp"]) for k in mfma)
    t1 = max(int(k["End_Timestamp"]) for k in mfma)
    out = []
    for k in kernels:
        a, b = int(k["Start_Timestamp"]), int(k["End_Timestamp"])
        if b <= t0 or a >= t1 or "zvc_pack" in k["Kernel_Name"] or "zvc_begin" in k["Kernel_Name"] or "zvc_end" in k["Kernel_Name"]:
            continue
        out.append(("compute", a, b))
    moved = {"d2h": 0, "h2d": 0}
    for c in copies:
        a, b = int(c["Start_Timestamp"]), int(c["End_Timestamp"])
        direction = c.get("Direction", "")
        kind = "d2h" if "DEVICE_TO_HOST" in direction else "h2d" if "HOST_TO_DEVICE" in direction else None
        if kind is None or b <= t0 or a >= t1:
            continue
        out.append((kind, a, b))
        moved[kind] += 1
    return out, moved


def main(argv):
    if len(argv) != 2:
        raise SystemExit(__doc__)
    intervals, moved = from_rocprof(argv[1])
    s = summarize(intervals)
    ms = lambda v: v / 1e6
    print("copies between the first and the last matrix-core kernel: %d device-to-host, %d host-to-device" % (moved["d2h"], moved["h2d"]))
    print("span %.1f ms, kernels busy %.1f ms, copies busy %.1f ms (device-to-host %.1f, host-to-device %.1f)" % (
        ms(s["span"]), ms(s["compute_busy"]), ms(s["copy_busy"]), ms(s["d2h_busy"]), ms(s["h2d_busy"])))
    print("copy time beside kernels %.1f ms = overlap fraction %s; exposed %.1f ms; both directions at once %.1f ms" % (
        ms(s["copy_beside_compute"]), "%.3f" % s["overlap_fraction"] if s["overlap_fraction"] is not None else "n/a",
        ms(s["copy_exposed"]), ms(s["duplex"])))


if __name__ == "__main__":
    main(sys.argv)
