"""Writes tests/golden/slicer_golden.json: inputs and outputs of the reference's own
KVWorker::DefaultSlicer (include/ps/kv_app.h:517-572) and FindRange (sarray.h:281-287).

Run in a container that has the reference tree: `make -C oracle ref` compiles the two
functions from the reference's headers into oracle/_ref/libpskv_ref.so, this script feeds
them the cases below and records what they return. The fixture holds data only.

    python tests/golden/make_slicer_golden.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, REPO)
from oracle import binding as orc  # noqa: E402

KMAX = (1 << 64) - 1


def stock_ranges(S):
    return [KMAX // S * i for i in range(S)], [KMAX // S * (i + 1) for i in range(S)]


def case(name, keys, rb, re, lens=None, nvals=0):
    ok, klo, khi, vlo, vhi, used, err = orc.ref_slice(np.array(keys, np.uint64), np.array(rb, np.uint64),
                                                      np.array(re, np.uint64),
                                                      None if lens is None else np.array(lens, np.int32), nvals)
    out = {"name": name, "keys": [int(k) for k in keys], "range_begin": [int(x) for x in rb],
           "range_end": [int(x) for x in re], "lens": None if lens is None else [int(x) for x in lens],
           "nvals": int(nvals), "ok": bool(ok)}
    if ok:
        out.update(used=[int(x) for x in used], key_lo=[int(x) for x in klo], key_hi=[int(x) for x in khi],
                   val_lo=[int(x) for x in vlo], val_hi=[int(x) for x in vhi])
    else:
        # keep only the CHECK text, not the stack trace
        line = [l for l in err.splitlines() if "Check failed" in l]
        out["check"] = line[0].split("Check failed:")[1].strip() if line else err[:200]
        out["check_line"] = int(line[0].split("kv_app.h:")[1].split(":")[0]) if line and "kv_app.h:" in line[0] else \
            (int(line[0].split("sarray.h:")[1].split(":")[0]) if line and "sarray.h:" in line[0] else 0)
    return out


def main():
    rng = np.random.default_rng(2024)
    cases = []
    rb4, re4 = stock_ranges(4)
    base = [0, 1, KMAX // 4 - 1, KMAX // 4, KMAX // 4 * 2 + 5, KMAX // 4 * 4 - 1]
    cases.append(case("s4_k2", base, rb4, re4, None, 12))
    cases.append(case("s4_lens", base, rb4, re4, [1, 0, 3, 2, 5, 1], 12))
    cases.append(case("s4_pull_no_vals", base, rb4, re4, None, 0))
    cases.append(case("s4_uncovered_top_key", base[:-1] + [KMAX - 3], rb4, re4, None, 6))
    cases.append(case("s4_vals_not_divisible", base, rb4, re4, None, 7))
    cases.append(case("s4_lens_size_mismatch", base, rb4, re4, [1, 0, 3, 2, 5], 12))
    cases.append(case("s4_lens_exceed_vals", base, rb4, re4, [1, 0, 3, 2, 5, 1], 11))
    cases.append(case("s4_lens_trailing_vals", base, rb4, re4, [1, 0, 3, 2, 5, 1], 20))
    cases.append(case("s4_empty_keys", [], rb4, re4, None, 0))
    cases.append(case("s4_empty_middle", [5, KMAX // 4 * 3 + 9], rb4, re4, [3, 4], 7))
    cases.append(case("s4_all_in_last", [KMAX // 4 * 3, KMAX // 4 * 3 + 1, KMAX // 4 * 4 - 1], rb4, re4, None, 3))
    gap = list(rb4)
    gap[2] += 1
    cases.append(case("s4_range_gap", base, gap, re4, None, 6))
    cases.append(case("sub_ranges_skip_front_k2", base, rb4[1:], re4[1:], None, 12))
    cases.append(case("sub_ranges_skip_front_lens", base, rb4[1:], re4[1:], [1, 0, 3, 2, 5, 1], 12))
    cases.append(case("s1_top_key_uncovered", [3, KMAX], [0], [KMAX], None, 2))
    cases.append(case("s1_all", [3, KMAX - 1], [0], [KMAX], None, 2))
    cases.append(case("negative_len", base, rb4, re4, [1, -1, 3, 2, 5, 1], 11))
    for S in (1, 2, 3, 7, 16):
        rb, re = stock_ranges(S)
        n = int(rng.integers(1, 40))
        keys = np.unique(rng.integers(0, re[-1], size=n, dtype=np.uint64)).tolist()
        lens = rng.integers(0, 9, size=len(keys)).tolist()
        cases.append(case("rand_s%d_lens" % S, keys, rb, re, lens, int(sum(lens))))
        cases.append(case("rand_s%d_k3" % S, keys, rb, re, None, 3 * len(keys)))
    find_range = []
    for arr, lo, hi in [([1, 3, 5, 7, 9], 2, 7), ([1, 3, 5, 7, 9], 0, 100), ([1, 3, 5, 7, 9], 7, 2),
                        ([1, 3, 5, 7, 9], 9, 10), ([], 0, 5), ([4, KMAX], KMAX, 0)]:
        b, e = orc.find_range(np.array(arr, np.uint64), lo, hi, use_ref=True)
        find_range.append({"arr": arr, "lower": lo, "upper": hi, "begin": b, "end": e})
    with open(os.path.join(HERE, "slicer_golden.json"), "w") as f:
        json.dump({"source": "ps::KVWorker<float>::DefaultSlicer and ps::FindRange compiled from the "
                             "reference headers (oracle/Makefile target `ref`)",
                   "slicer": cases, "find_range": find_range}, f, indent=1)
    print("wrote", len(cases), "slicer cases and", len(find_range), "FindRange cases")


if __name__ == "__main__":
    main()
