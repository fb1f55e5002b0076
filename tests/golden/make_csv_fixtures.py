#!/usr/bin/env python3
"""Extracts the host-validation test tables of the reference into JSON fixtures.

The reference keeps its operator API tests as CSV rows (one row = operator
param JSON + input dtypes/formats/shapes + output dtype/shape + the expected
status, tagged C: for CreateOperation, I: for InferShape, S: for Setup):
    tests/apitest/opstest/csv/paged_attention.csv
    tests/apitest/opstest/csv/reshape_and_cache.csv
    tests/apitest/opstest/csv/multi_latent_attention.csv
    tests/apitest/opstest/csv/block_copy.csv
    tests/apitest/opstest/csv/paged_cache_load.csv
    tests/apitest/opstest/csv/norm_rope_reshape.csv
    tests/apitest/opstest/csv/rope.csv
    tests/apitest/opstest/csv/elewise.csv (the rows of the two per-channel quantiser types)
    tests/apitest/opstest/csv/reshape_and_cache_omni.csv
Those rows are data, not code. This script copies the rows written for the
Ascend910B feature set (the one this library mirrors) into
    tests/golden/paged_attention_cases.json
    tests/golden/reshape_and_cache_cases.json
    tests/golden/multi_latent_attention_cases.json
    tests/golden/block_copy_cases.json
    tests/golden/paged_cache_load_cases.json
    tests/golden/norm_rope_reshape_cases.json
    tests/golden/rope_cases.json
    tests/golden/elewise_cases.json
    tests/golden/reshape_and_cache_omni_cases.json
so the parity tests can run where the reference tree is absent.

Run from the repository root in a container that has /root/reference:
    python3 tests/golden/make_csv_fixtures.py
"""
import csv
import json
import os
import sys

REF = os.environ.get("ATB_REFERENCE", "/root/reference")
HERE = os.path.dirname(os.path.abspath(__file__))


def split(field):
    return [x.strip() for x in field.split(";") if x.strip() != ""]


def shapes(field):
    out = []
    for s in split(field):
        out.append([int(x) for x in s.split(",") if x.strip() != ""])
    return out


def convert(name, also_untagged=False, keep=None):
    path = os.path.join(REF, "tests/apitest/opstest/csv", name + ".csv")
    rows = list(csv.reader(open(path, newline=""), delimiter="|"))
    header = [h.strip() for h in rows[0]]
    cases = []
    for line_no, row in enumerate(rows[1:], start=2):
        if not any(c.strip() for c in row):
            continue
        d = {h: v.strip() for h, v in zip(header, row)}
        # (a creation-only row may leave every column after the param empty, the product tag included,
        # and a row may name several products, or none when it holds for all of them)
        tags = [t.strip() for t in d.get("SocVersion", "").split(",") if t.strip()]
        if "Ascend910B" not in tags and not (also_untagged and not tags):
            continue
        if keep is not None and not keep(json.loads(d["OpParam"])):
            continue
        # OutNum is what the harness hands to the operation (BlockCopy lists two output columns but takes none)
        n_out = int(d["OutNum"]) if d.get("OutNum", "").strip().isdigit() else None
        cases.append({
            "csv_line": line_no,
            "case": int(d["CaseNum"]),
            "name": d["CaseName"],
            "op": d["OpName"],
            "param": json.loads(d["OpParam"]),
            "in_dtypes": split(d["InDType"]),
            "in_formats": split(d["InFormat"]),
            "in_shapes": shapes(d["InShape"]),
            "out_dtypes": split(d["OutDType"])[:n_out],
            "out_formats": split(d["OutFormat"])[:n_out],
            "out_shapes": shapes(d["OutShape"])[:n_out],
            "expected": d["ExpectedError"],
        })
    out = os.path.join(HERE, name + "_cases.json")
    with open(out, "w") as f:
        json.dump({"source": "tests/apitest/opstest/csv/%s.csv (rows with SocVersion Ascend910B)" % name,
                   "cases": cases}, f, indent=1)
    print(out, len(cases), "cases")


if __name__ == "__main__":
    if not os.path.isdir(REF):
        sys.exit("reference tree not found at " + REF)
    convert("paged_attention")
    convert("reshape_and_cache")
    convert("multi_latent_attention")
    convert("block_copy")
    convert("paged_cache_load")
    convert("norm_rope_reshape", also_untagged=True)
    convert("rope", also_untagged=True)
    convert("elewise", also_untagged=True, keep=lambda p: p.get("elewiseType") in (17, 18))
    convert("reshape_and_cache_omni")
