"""L2-miss traffic of the step's dense products, from hardware counters.

    python bench.py --workload gemm-traffic          # under rocprofv3 --pmc FETCH_SIZE, then --pmc WRITE_SIZE
    python -m cacti_amd.gemm_traffic <fetch counter_collection.csv> <write counter_collection.csv>

writes cacti_amd/gemm_traffic.json: per timing label of a product the mean FETCH_SIZE and WRITE_SIZE of
its launches (KiB per dispatch; a product that runs as two launches adds them) and the bytes they stand
for, bytes = (FETCH_FACTOR * FETCH_SIZE + WRITE_FACTOR * WRITE_SIZE) * 1024: a streaming copy kernel of
known size reads FETCH_SIZE = half its bytes and WRITE_SIZE = its bytes on this device.  The file also
records the SHA-256 of csrc/gemm_mfma.hip; load_current() returns the table only while that source is
the one the figures were taken on.
"""
import csv
import hashlib
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
TABLE = os.path.join(HERE, "gemm_traffic.json")
KERNEL_SOURCE = os.path.join(HERE, "csrc", "gemm_mfma.hip")
LAUNCHES = 4
FETCH_FACTOR, WRITE_FACTOR = 2.0, 1.0

# timing labels of the dense products of one 3B-shaped step (S = 2048, D = 3200, F = 8640, V = 32000)
STEP_PRODUCTS = [
    "matmul[NT,1x2048x3200x3200]", "matmul[NT,1x2048x8640x3200]", "matmul[NT,1x2048x3200x8640]",
    "matmul[NT,1x2048x32000x3200]",
    "matmul[NN,1x2048x3200x3200]", "matmul[NN,1x2048x3200x3200,acc]", "matmul[NN,1x2048x3200x8640]",
    "matmul[NN,1x2048x3200x8640,acc]", "matmul[NN,1x2048x8640x3200]", "matmul[NN,1x2048x3200x32000]",
    "matmul[TN,1x3200x3200x2048]", "matmul[TN,1x8640x3200x2048]", "matmul[TN,1x3200x8640x2048]",
    "matmul[TN,1x32000x3200x2048]",
]


def source_hash():
    with open(KERNEL_SOURCE, "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()


def load_current():
    """{label: {"fetch_kib", "write_kib", "bytes", "launches_per_product"}} if the table was taken on the
    kernels as they are now, else None."""
    if not os.path.exists(TABLE):
        return None
    with open(TABLE) as f:
        t = json.load(f)
    return t["products"] if t.get("kernel_source_sha256") == source_hash() else None


def _dispatches(path):
    """Counter value per GEMM dispatch, in dispatch order."""
    rows = []
    with open(path) as f:
        for r in csv.DictReader(f):
            if "gemm_mfma_kernel" in r["Kernel_Name"]:
                rows.append((int(r["Dispatch_Id"]), float(r["Counter_Value"]), r["Kernel_Name"]))
    rows.sort()
    return rows


def build(fetch_csv, write_csv, launches_per_product):
    """launches_per_product: {label: 1 or 2} (2: the columns beyond the full rounds go to a second kernel)."""
    f, w = _dispatches(fetch_csv), _dispatches(write_csv)
    want = sum(LAUNCHES * launches_per_product[l] for l in STEP_PRODUCTS)
    assert len(f) == want and len(w) == want, "expected %d GEMM dispatches, found %d / %d" % (want, len(f), len(w))
    products, i = {}, 0
    for label in STEP_PRODUCTS:
        n = LAUNCHES * launches_per_product[label]
        fk = sum(v for _, v, _ in f[i:i + n]) / LAUNCHES
        wk = sum(v for _, v, _ in w[i:i + n]) / LAUNCHES
        products[label] = {"fetch_kib": fk, "write_kib": wk, "launches_per_product": launches_per_product[label],
                           "kernel": f[i][2], "bytes": (FETCH_FACTOR * fk + WRITE_FACTOR * wk) * 1024.0}
        i += n
    return {"kernel_source_sha256": source_hash(), "fetch_factor": FETCH_FACTOR, "write_factor": WRITE_FACTOR,
            "launches_averaged": LAUNCHES, "products": products}


def main(argv):
    if len(argv) != 3:
        sys.exit(__doc__)
    sys.path.insert(0, os.path.dirname(HERE))
    import bench
    per = {l: 2 if bench.is_split(l) else 1 for l in STEP_PRODUCTS}
    t = build(argv[1], argv[2], per)
    with open(TABLE, "w") as f:
        json.dump(t, f, indent=1, sort_keys=True)
        f.write("\n")
    for l in STEP_PRODUCTS:
        p = t["products"][l]
        print("%-36s FETCH %9.0f KiB  WRITE %9.0f KiB  -> %7.1f MB" % (l, p["fetch_kib"], p["write_kib"], p["bytes"] / 1e6))


if __name__ == "__main__":
    main(sys.argv)
