#!/usr/bin/env python3
"""Writes tests/golden/ref_signatures.json from the reference's own nvprof traces.

The reference holds no source of the kernels it fuses; the only place it pins each
original kernel's argument list is the kernel-name column of scripts/data/ml-event.csv and
scripts/data/ethminer_event.csv.  This script reads those two data files (as text) and
records, per kernel, the file:line, the signature string as nvprof printed it, the number
of parameters, and the class of each parameter where nvprof's demangler left it readable
("ptr", "scalar", "uint2"; "opaque" for accessor / TensorInfo structs and for the positions
its substitution decoding garbled).  Run in the container that has /root/reference:

    python3 tests/golden/make_ref_signatures.py
"""
import csv
import json
import os
import re

REF = "/root/reference/scripts/data"
WANT = {  # kernel -> (file, regex that selects the native kernel's row)
    "im2col_kernel": ("ml-event.csv", r"^void at::native::im2col_kernel<float>\("),
    "MaxPoolForward": ("ml-event.csv", r"^void at::native::MaxPoolForward<float, float>\("),
    "batch_norm_collect_statistics_kernel":
        ("ml-event.csv", r"^void at::native::batch_norm_collect_statistics_kernel<at::native::InvStd, float, float, float, int>\("),
    "upsample_bilinear2d_out_frame": ("ml-event.csv", r"::upsample_bilinear2d_out_frame<float, float>\(int"),
    "kernelHistogram1D": ("ml-event.csv", r"^_ZN2at6native17kernelHistogram1DIfflLi1ELi2ELin1E"),
    "ethash_search": ("ethminer_event.csv", r"^ethash_search\("),
    "sha256d_gpu_hash_shared": ("ethminer_event.csv", r"::sha256d_gpu_hash_shared\("),
    "blake2b_gpu_hash": ("ethminer_event.csv", r"::blake2b_gpu_hash\(unsigned int, unsigned int, unsigned int\*, uint2\)$"),
    "sia_blake2b_gpu_hash": ("ethminer_event.csv", r"^sia_blake2b_gpu_hash\("),
}
SCALARS = {"int", "long", "float", "bool", "unsigned int", "unsigned long"}


def split_params(sig):
    """Top-level comma split of the last parenthesised group."""
    depth, start, end = 0, None, None
    for i in range(len(sig) - 1, -1, -1):
        if sig[i] == ")":
            if depth == 0:
                end = i
            depth += 1
        elif sig[i] == "(":
            depth -= 1
            if depth == 0:
                start = i
                break
    body, out, cur, d = sig[start + 1:end], [], "", 0
    for ch in body:
        if ch in "<(":
            d += 1
        elif ch in ">)":
            d -= 1
        if ch == "," and d == 0:
            out.append(cur.strip())
            cur = ""
        else:
            cur += ch
    out.append(cur.strip())
    return out


def classify(p):
    if p in SCALARS:
        return "scalar"
    if p == "uint2":
        return "uint2"
    if p.endswith("*"):
        return "ptr"
    return "opaque"


def main():
    out = {}
    for kernel, (fname, pattern) in WANT.items():
        with open(os.path.join(REF, fname), newline="") as f:
            for lineno, row in enumerate(csv.reader(f), start=1):
                if len(row) > 1 and re.search(pattern, row[1]):
                    sig = row[1]
                    entry = {"source": f"scripts/data/{fname}:{lineno}", "signature": sig}
                    if sig.startswith("_Z"):
                        # Itanium-mangled only: parameters after the template arguments are
                        # TensorInfo, TensorInfo, TensorInfo, i, float, float, long, Op
                        entry["arity"] = 8
                        entry["params"] = ["opaque", "opaque", "opaque", "scalar", "scalar", "scalar", "scalar", "opaque"]
                        entry["note"] = "nvprof left this name mangled; decoded by hand from ...EEvNS_4cuda6detail10TensorInfoIS9_T1_EESK_NSI_IT0_SJ_EEiSL_SL_SJ_T6_"
                    else:
                        ps = split_params(sig)
                        entry["arity"] = len(ps)
                        classes = [classify(p) for p in ps]
                        # nvprof's demangler mis-resolves substitutions in long template signatures: from
                        # the first parameter that merely repeats an earlier struct parameter on, the
                        # printed types are not trustworthy (only the count is)
                        for i, prm in enumerate(ps):
                            if classes[i] == "opaque" and prm in ps[:i]:
                                classes[i:] = ["opaque"] * (len(ps) - i)
                                entry["note"] = f"parameter types garbled by nvprof from position {i} on; arity only"
                                break
                        entry["params"] = classes
                    out[kernel] = entry
                    break
            else:
                raise SystemExit(f"{kernel}: no row matches in {fname}")
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_signatures.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    print("wrote", path)


if __name__ == "__main__":
    main()
