#!/usr/bin/env python3
"""Writes the fixtures partition_*.json in this folder.

The reference ships no known-answer data for its partition (its only check is eQcheck on y), so
these vectors come from a third, deliberately naive restatement of the canonical partition:
plain Python lists and sorted(), written from the reference's host code alone
(test/test_autotc_spmv.cpp:1106-1345 cascade, :502-585 and :718-978 tile format, :129-250
residual) and sharing no code with the C oracle or the library.  Values and x are small integers,
so every sum is exact in binary64 and binary16 alike and y is known exactly.

    python3 tests/golden/make_golden.py        # rewrites the fixtures (deterministic)
"""
import json
import os
import random
import struct

HERE = os.path.dirname(os.path.abspath(__file__))


def f32(v):
    return struct.unpack("f", struct.pack("f", v))[0]


def threshold(nnz, tau):
    """(int)((float)nnz * tau) with tau a float (test_autotc_spmv.cpp:1131,1249)."""
    return int(f32(f32(float(nnz)) * f32(tau)))


def prefix_count(counts, order, target):
    """Smallest k >= 1 whose first k counts (in `order`) add up to at least target (:1133-1141)."""
    total = 0
    for k, i in enumerate(order):
        total += counts[i]
        if total >= target:
            return k + 1, total
    raise ValueError("threshold not reachable: not a case for these fixtures")


def partition(rows, cols, row_ptr, col_ind, val, tau_c, tau_r, frag_k):
    frag_m = 8
    entries = []  # (row, col, value) in the order of the input
    for r in range(rows):
        for p in range(row_ptr[r], row_ptr[r + 1]):
            entries.append((r, col_ind[p], val[p]))
    nnz = len(entries)
    # column pass
    ccount = [0] * cols
    for _, c, _ in entries:
        ccount[c] += 1
    desc_col = sorted(range(cols), key=lambda c: (-ccount[c], c))
    d_cols, nnz_col_d = prefix_count(ccount, desc_col, threshold(nnz, tau_c))
    dense_rank = {c: j for j, c in enumerate(desc_col[:d_cols])}
    new_array = [c for c in range(cols) if c not in dense_rank]
    sparse_rank = {c: j for j, c in enumerate(new_array)}
    # per row: the dense-column part and the sparse-column part, ascending new column id, equal
    # ids in the order of the input (sorted() is stable)
    d_part = [sorted([(dense_rank[c], v) for r, c, v in entries if r == i and c in dense_rank], key=lambda t: t[0])
              for i in range(rows)]
    s_part = [sorted([(sparse_rank[c], v) for r, c, v in entries if r == i and c in sparse_rank], key=lambda t: t[0])
              for i in range(rows)]
    # row pass
    rcount = [len(d) for d in d_part]
    desc_row = sorted(range(rows), key=lambda r: (-rcount[r], r))
    d_rows, nnz_row_d = prefix_count(rcount, desc_row, threshold(nnz, tau_r))
    r_id = desc_row[:d_rows]
    new_array_ = [r for r in range(rows) if r not in set(r_id)]
    dd = [d_part[r] for r in r_id]
    # tile format
    chunk_num = (d_rows + frag_m - 1) // frag_m
    chunk_ptr, atox, frag_bit, tc_val, frag_ptr = [0], [], [], [], [0]
    for w in range(chunk_num):
        window = dd[w * frag_m:(w + 1) * frag_m]
        used = sorted({c for row in window for c, _ in row})
        nfrag = (len(used) + frag_k - 1) // frag_k
        chunk_ptr.append(chunk_ptr[-1] + nfrag)
        atox += used + [0] * (nfrag * frag_k - len(used))
        rank = {c: j for j, c in enumerate(used)}
        cells = [dict() for _ in range(nfrag)]  # bit -> value; a later entry of the same cell replaces the earlier
        for lr, row in enumerate(window):
            for c, v in row:
                cells[rank[c] // frag_k][lr * frag_k + rank[c] % frag_k] = v
        for cell in cells:
            bits = 0
            for b in sorted(cell):
                bits |= 1 << b
                tc_val.append(cell[b])
            frag_bit.append(bits)
            frag_ptr.append(frag_ptr[-1] + len(cell))
    # residual
    cd_ptr, cd_col, cd_val = [0], [], []
    dense_rows = set(r_id)
    for i in range(rows):
        for j, v in s_part[i]:
            cd_col.append(d_cols + j)
            cd_val.append(v)
        if i not in dense_rows:
            for j, v in d_part[i]:
                cd_col.append(j)
                cd_val.append(v)
        cd_ptr.append(len(cd_col))
    return {
        "dCols": d_cols, "sCols": cols - d_cols, "nnzColD": nnz_col_d, "dRows": d_rows, "sRows": rows - d_rows,
        "nnzRowD": nnz_row_d, "chunkNum": chunk_num, "totalTcFrags": chunk_ptr[-1], "nnzCD": len(cd_col),
        "descColId": desc_col, "newArray": new_array, "rId": r_id, "newArray_": new_array_,
        "ddRowPtr": [0] + [sum(len(r) for r in dd[:i + 1]) for i in range(d_rows)],
        "ddColInd": [c for row in dd for c, _ in row], "ddVal": [v for row in dd for _, v in row],
        "chunkPtr": chunk_ptr, "sparse_AToX_index": atox, "fragPtr": frag_ptr,
        "fragBit": ["%x" % b for b in frag_bit], "tcVal": tc_val,
        "cdRowPtr": cd_ptr, "cdColInd": cd_col, "cdVal": cd_val,
    }


def product(rows, row_ptr, col_ind, val, x):
    return [sum(val[p] * x[col_ind[p]] for p in range(row_ptr[r], row_ptr[r + 1])) for r in range(rows)]


def random_matrix(rng, rows, cols, density, sorted_rows=True, twice=0.0):
    row_ptr, col_ind = [0], []
    for _ in range(rows):
        c = [j for j in range(cols) if rng.random() < density]
        c += [rng.choice(c) for _ in c if rng.random() < twice]  # a column named twice
        if not sorted_rows:
            rng.shuffle(c)
        col_ind += c
        row_ptr.append(len(col_ind))
    val = [rng.choice([-3, -2, -1, 1, 2, 3]) for _ in col_ind]
    return row_ptr, col_ind, val


def cases():
    rng = random.Random(20240611)
    out = []
    # 1: small enough to follow by hand: a 12x12 band with one full column and one full row
    rows = cols = 12
    row_ptr, col_ind = [0], []
    for r in range(rows):
        c = sorted({r, (r + 1) % cols, 5} | (set(range(cols)) if r == 3 else set()))
        col_ind += c
        row_ptr.append(len(col_ind))
    out.append(("band12", rows, cols, row_ptr, col_ind, [1 + (p % 5) for p in range(len(col_ind))], 0.5, 0.25))
    # 2: all counts equal (a circulant): ties keep the ascending order
    rows = cols = 16
    row_ptr, col_ind = [0], []
    for r in range(rows):
        col_ind += sorted({r, (r + 3) % cols, (r + 7) % cols})
        row_ptr.append(len(col_ind))
    out.append(("circulant16", rows, cols, row_ptr, col_ind, [1 + (p % 3) for p in range(len(col_ind))], 0.5, 0.5))
    # 3, 4: random, several chunks, the usual case
    rp, ci, va = random_matrix(rng, 37, 37, 0.18)
    out.append(("random37", 37, 37, rp, ci, va, 0.6, 0.4))
    rp, ci, va = random_matrix(rng, 45, 29, 0.25)
    out.append(("tall45x29", 45, 29, rp, ci, va, 0.75, 0.5))
    # 5: rows in any column order, columns named twice, everything extracted
    rp, ci, va = random_matrix(rng, 30, 30, 0.2, sorted_rows=False, twice=0.3)
    out.append(("twice30", 30, 30, rp, ci, va, 1.0, 1.0))
    # 6: tau_r = 0: exactly one dense row
    rp, ci, va = random_matrix(rng, 20, 20, 0.3)
    out.append(("onerow20", 20, 20, rp, ci, va, 0.5, 0.0))
    return out


def main():
    rng = random.Random(7)
    for name, rows, cols, row_ptr, col_ind, val, tau_c, tau_r in cases():
        x = [rng.choice([-2, -1, 0, 1, 2]) for _ in range(cols)]
        fixture = {
            "name": name, "rows": rows, "cols": cols, "rowPtr": row_ptr, "colInd": col_ind, "val": val,
            "tau_c": tau_c, "tau_r": tau_r, "x": x, "y": product(rows, row_ptr, col_ind, val, x),
            "f64": partition(rows, cols, row_ptr, col_ind, val, tau_c, tau_r, 4),
            "f16": partition(rows, cols, row_ptr, col_ind, val, tau_c, tau_r, 8),
        }
        with open(os.path.join(HERE, "partition_%s.json" % name), "w") as f:
            json.dump(fixture, f, separators=(",", ":"))
            f.write("\n")
        print(name, "rows", rows, "nnz", len(col_ind), "dCols", fixture["f64"]["dCols"], "dRows", fixture["f64"]["dRows"],
              "frags f64/f16", fixture["f64"]["totalTcFrags"], fixture["f16"]["totalTcFrags"])


if __name__ == "__main__":
    main()
