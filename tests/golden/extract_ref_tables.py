#!/usr/bin/env python3
"""Extracts the parameter tables of the reference's gemm / pack / cvt test
suites into ref_tables.json (data only: one record of numbers per test row).

Run in a container that has the SKL checkout:
    python tests/golden/extract_ref_tables.py [/root/reference]
The JSON is committed; tests read the JSON, never the checkout.
"""
import json
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
SUITES = [
    "test/gemm/rvv/skl_gemm_i8_i8_i32_zve32x.c",
    "test/gemm/rvv/skl_gemm_i8_i8_i32_zve32x_x390.c",
    "test/gemm/rvv/skl_gemm_bf16_bf16_f32_zvfbfwma.c",
    "test/gemm/rvv/skl_gemm_bf16_bf16_f32_zvfbfwma_x390.c",
    "test/gemm/rvv/skl_gemm_f16_f16_f32_zvfh.c",
    "test/gemm/rvv/skl_gemm_f16_f16_f32_zvfh_x390.c",
    "test/gemm/rvv/skl_gemm_f16_f16_f16_zvfh.c",
    "test/gemm/rvv/skl_gemm_f16_f16_f16_zvfh_x390.c",
    "test/gemm/rvv/skl_gemm_f32_f32_f32_zve32f.c",
    "test/gemm/rvv/skl_gemm_f32_f32_f32_zve32f_x390.c",
    "test/gemm/rvv/skl_gemm_f64_f64_f64_zve64d.c",
    "test/gemm/rvv/skl_gemm_f64_f64_f64_zve64d_x390.c",
    "test/gemm/xsfmm/skl_gemm_i8c_i8_i32_xsfmm32a8i.c",
    "test/gemm/xsfmm/skl_gemm_bf16c_bf16_f32_xsfmm32a16f.c",
    "test/gemm/xsfmm/skl_gemm_f16c_f16_f32_xsfmm32a16f.c",
    "test/gemm/xsfmm/skl_gemm_f8e4m3c_f8e4m3_f32_xsfmm32a8f.c",
    "test/gemm/xsfmm/skl_gemm_f8e5m2c_f8e5m2_f32_xsfmm32a8f.c",
    "test/gemm/xsfmm/skl_gemm_f32c_f32_f32_xsfmm32a32f.c",
    "test/gemm/xsfmm/skl_gemm_i8rcptex1c_i8rcp1xte_i32rcptexterc_xsfmm32a8i.c",
    "test/gemm/xsfmm/skl_gemm_bf16rcptex1c_bf16rcp1xte_f32rcptexterc_xsfmm32a16f.c",
    "test/gemm/xsfmm/skl_gemm_f16rcptex1c_f16rcp1xte_f32rcptexterc_xsfmm32a16f.c",
    "test/gemm/xsfmm/skl_gemm_f8e4m3rcptex1c_f8e4m3rcp1xte_f32rcptexterc_xsfmm32a8f.c",
    "test/gemm/xsfmm/skl_gemm_f8e5m2rcptex1c_f8e5m2rcp1xte_f32rcptexterc_xsfmm32a8f.c",
    "test/gemm/xsfmm/skl_gemm_f32rcptex1c_f32rcp1xte_f32rcptexterc_xsfmm32a32f.c",
    "test/gemm/xsfvqdotq/skl_gemm_i8rcp1x4_i8p4x1c_i32_xsfvqdotq.c",
    "test/pack/rvv/skl_pack_e8rc_e8rcprc_zve32x.c",
    "test/pack/rvv/skl_pack_e16rc_e16rcprc_zve32x.c",
    "test/pack/rvv/skl_pack_e32rc_e32rcprc_zve32x.c",
    "test/pack/rvv/skl_unpack_e8rcprc_e8rc_zve32x.c",
    "test/pack/rvv/skl_transpose_e8_zve32x.c",
    "test/pack/rvv/skl_transpose_e16_zve32x.c",
    "test/pack/rvv/skl_transpose_e32_zve32x.c",
    "test/pack/xsfmm/skl_pack_e16_e16rcptex1c_xsfmmbase.c",
    "test/pack/xsfmm/skl_pack_e32_e32rcptex1c_xsfmmbase.c",
    "test/pack/xsfmm/skl_transpose_e8_xsfmmbase.c",
    "test/pack/xsfmm/skl_transpose_e16_xsfmmbase.c",
    "test/pack/xsfmm/skl_transpose_e32_xsfmmbase.c",
    "test/cvt/cvt_f32_f8_zvfofp8min.c",
    "test/cvt/cvt_bf16_f8_zvfofp8min_zvfbfmin.c",
    "test/cvt/cvt_f8_bf16_zvfofp8min.c",
    "test/cvt/cvt_f4_f8_zvfofp4min.c",
]
# Symbols the tables use; the tile edge is 64 in the reference's test setup
# (cmake/riscv.cmake:22 selects xsfmm64t).
ENV = {"__riscv_min_xsfmm_te": 64, "SKL_XSFMM_TE": 64, "ETE": 64, "TE": 64, "true": 1, "false": 0, "NULL": 0}

REC = re.compile(r"\{\s*((?:TEST|BENCH)\w*)\s*,(.*?)\}", re.S)
FIELD = re.compile(r"\.(\w+)\s*=\s*([^,}]+)")


def evaluate(expr, unknown):
    expr = expr.strip().replace("(size_t)", "").replace("(_Float16)", "").strip()
    if re.fullmatch(r"[\d.]+[fFuUlL]*", expr):
        expr = expr.rstrip("fFuUlL")
    try:
        return eval(expr, {"__builtins__": {}}, ENV)
    except Exception:
        unknown.add(expr)
        return expr


def main():
    out = {}
    unknown = set()
    for rel in SUITES:
        path = os.path.join(REF, rel)
        text = open(path).read()
        # only the table: from "tests[] = {" to the matching "};"
        start = text.index("tests[] = {")
        end = text.index("};", start)
        table = text[start:end]
        base_line = text[:start].count("\n") + 1
        rows = []
        for m in REC.finditer(table):
            rec = {"kind": m.group(1), "line": base_line + table[:m.start()].count("\n")}
            for f in FIELD.finditer(m.group(2)):
                rec[f.group(1)] = evaluate(f.group(2), unknown)
            rows.append(rec)
        out[rel] = rows
        print(f"{rel}: {len(rows)} rows")
    if unknown:
        print("unevaluated expressions:", sorted(unknown))
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_tables.json")
    with open(dst, "w") as fh:
        json.dump(out, fh, indent=0, sort_keys=True)
    print("wrote", dst)


if __name__ == "__main__":
    main()
