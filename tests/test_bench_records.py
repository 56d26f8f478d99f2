"""bench.py quotes fabric-traffic figures from the committed rocprofv3 summaries; this ties the two together, so that a
kernel change which moves the counters cannot leave the JSON line quoting stale bytes."""
import os
import re
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GATHER_KERNELS = {"spmm": ("spmm_items_kernel",), "sddmm": ("sddmm_tiled_kernel", "sddmm_coo_kernel", "sddmm_csr_kernel")}


def _parse(path):
    text = open(path).read()
    head = re.search(r"workload (\S+) .*?F=(\d+)", text)
    spmm = re.search(r"SpMM [\d.]+ ms \((\d+) partitions x (\d+) tiles", text)
    sddmm = re.search(r"SDDMM [\d.]+ ms \(\w+, (\d+) partitions x (\d+) tiles", text)
    table = text[text.index("Per launch, after calibration:"):]
    rows = {}
    for line in table.splitlines()[2:]:
        m = re.match(r"(\S.*?)\s+([\d.]+)\s+([\d.]+)\s+[\d.]+\s+\d+%", line)
        if not m:
            break
        rows[m.group(1).strip()] = float(m.group(2)) + float(m.group(3))
    return dict(workload=head.group(1), F=int(head.group(2)), spmm=tuple(int(v) for v in spmm.groups()),
                sddmm=tuple(int(v) for v in sddmm.groups()), rows=rows)


def test_stored_traffic_figures_match_their_summaries():
    import bench
    assert bench.MEASURED_TRAFFIC, "no stored traffic figures"
    for (op, workload, F, parts, tiles), (nbytes, summary) in bench.MEASURED_TRAFFIC.items():
        path = os.path.join(ROOT, summary)
        assert os.path.exists(path), "%s names a summary that is not committed: %s" % ((op, workload, F), summary)
        rec = _parse(path)
        assert (rec['workload'], rec['F']) == (workload, F), (summary, rec['workload'], rec['F'])
        # the tiling the summary was taken at is the one the figure is stored for (0 tiles = the kernel's own single tile)
        assert rec[op] == (parts, max(tiles, 1)), "%s: summary taken at %s, figure stored for %s" % (summary, rec[op], (parts, tiles))
        hits = [gb for name, gb in rec['rows'].items() if name.startswith(GATHER_KERNELS[op])]
        assert len(hits) == 1, "%s: %d gather-kernel rows for %s" % (summary, len(hits), op)
        assert abs(hits[0] * 1e9 - nbytes) <= 0.01 * nbytes, \
            "%s %s F=%d: bench.py stores %.3g bytes, the summary's table gives %.4g GB" % (op, workload, F, nbytes, hits[0])


def test_byte_models():
    """The compulsory-traffic models of bench.py, on a case small enough to count by hand."""
    import bench
    # 3 x 4 adjacency with 5 stored elements, F = 2: indptr 4 ints, 5 column ids + 5 weights, X 4 x 2, out 3 x 2
    assert bench.spmm_bytes(3, 4, 5, 2) == 4 * 4 + 8 * 5 + 4 * 4 * 2 + 4 * 3 * 2
    # square, n = 3, 5 edges, F = 2, 2 heads: CSR order reads indptr + column ids, COO order row + col
    assert bench.sddmm_bytes(3, 5, 2, 2, csr=True) == 4 * 4 + 4 * 5 + 8 * 3 * 2 + 4 * 5 * 2
    assert bench.sddmm_bytes(3, 5, 2, 1, csr=False) == 8 * 5 + 8 * 3 * 2 + 4 * 5
