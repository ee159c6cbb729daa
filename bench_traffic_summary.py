"""Turns two rocprofv3 counter passes of `bench.py --calibration-copy` into the memory-traffic
summary that `bench.py` reads its `roofline.traffic` figure from.

    python bench_traffic_summary.py FETCH_DIR WRITE_DIR > summary.txt

FETCH_DIR / WRITE_DIR: output folders of
    rocprofv3 --pmc FETCH_SIZE --output-format csv -d FETCH_DIR -o run -- \
        python3 bench.py --steps 3 --warmup 1 --no-cpu-baseline --calibration-copy
and the same with WRITE_SIZE.  The calibration dispatches (plain elementwise copies of the
input tensor, bytes known) give the bytes one count stands for; every other kernel's average
count per dispatch is scaled by it.  Lines that start with '@' are the machine-readable part:
the hash of the kernel source the run was made with, and per timed C-ABI call the kernel that
did its work with the bytes it read and wrote per launch.
"""
import collections
import csv
import glob
import hashlib
import os
import re
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
KERNEL_SOURCE = "mappedconvolutions_amd/csrc/mcx_conv_mfma.hip"
COPY_BYTES = 8 * 64 * 256 * 512 * 4  # one calibration dispatch reads and writes the input once


def source_hash():
    with open(os.path.join(ROOT, KERNEL_SOURCE), "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()


def short_name(name):
    name = name.replace("(anonymous namespace)::", "").replace("void mcx::", "")
    name = re.sub(r"\(.*", "", name)
    return name.replace(", ", ",")


def per_kernel(folder, counter):
    """{kernel: [count per dispatch]} and the list of calibration counts."""
    files = glob.glob(os.path.join(folder, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        sys.exit("no counter_collection.csv under " + folder)
    counts, copies = collections.defaultdict(list), []
    for row in csv.DictReader(open(files[0])):
        if row["Counter_Name"] != counter:
            continue
        value = float(row["Counter_Value"])
        name = row["Kernel_Name"]
        if "elementwise_kernel" in name:
            if int(row["Grid_Size"]) * 4 >= COPY_BYTES // 16:  # the whole-tensor copies only
                copies.append(value)
            continue
        if "mcx::" in name:
            counts[short_name(name)].append(value)
    return counts, copies


def label_of(kernel):
    """The timed C-ABI call whose work this kernel does (None: a helper kernel)."""
    if kernel.startswith("weight_grad_mfma_kernel<"):
        return "conv_backward_weight"
    m = re.match(r"gather_product_mfma_kernel<\w+,(\d+),(\d+),", kernel)
    if m:  # the forward resolves the four bilinear corners itself; the input gradient reads a
        # packed transposed map of one pair per slot
        return "conv_forward" if m.group(1) == "4" else "conv_backward_input"
    return None


def main(argv):
    if len(argv) != 2:
        sys.exit(__doc__)
    fetch, fcopies = per_kernel(argv[0], "FETCH_SIZE")
    write, wcopies = per_kernel(argv[1], "WRITE_SIZE")
    if not fcopies or not wcopies:
        sys.exit("no calibration dispatch found: run bench.py with --calibration-copy")
    fscale = COPY_BYTES / (sum(fcopies) / len(fcopies))
    wscale = COPY_BYTES / (sum(wcopies) / len(wcopies))
    print("Calibration: %d + %d copy dispatches of %d bytes each way;" %
          (len(fcopies), len(wcopies), COPY_BYTES))
    print("  one FETCH_SIZE count = %.1f bytes, one WRITE_SIZE count = %.1f bytes" %
          (fscale, wscale))
    print()
    print("%-58s %8s %12s %12s %10s %10s" % ("kernel (average per dispatch)", "launches",
                                             "FETCH_SIZE", "WRITE_SIZE", "read MB", "written MB"))
    rows = []
    for k in sorted(set(fetch) | set(write)):
        f = sum(fetch.get(k, [0])) / max(len(fetch.get(k, [])), 1)
        w = sum(write.get(k, [0])) / max(len(write.get(k, [])), 1)
        rows.append((k, len(fetch.get(k, [])), f, w, f * fscale, w * wscale))
    rows.sort(key=lambda r: -(r[4] + r[5]))
    for k, n, f, w, rb, wb in rows:
        print("%-58s %8d %12.0f %12.0f %10.1f %10.1f" % (k[:58], n, f, w, rb / 1e6, wb / 1e6))
    print()
    print("@source sha256=%s file=%s" % (source_hash(), KERNEL_SOURCE))
    best = {}
    for k, n, f, w, rb, wb in rows:
        lab = label_of(k)
        if lab and (lab not in best or rb + wb > best[lab][1] + best[lab][2]):
            best[lab] = (k, rb, wb)  # of two launched variants, the one that did the work
    for lab, (k, rb, wb) in sorted(best.items()):
        print('@traffic label=%s kernel="%s" read_bytes=%d written_bytes=%d' % (lab, k, rb, wb))


if __name__ == "__main__":
    main(sys.argv[1:])
