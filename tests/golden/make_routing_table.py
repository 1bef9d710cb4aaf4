"""Writes tests/golden/routing_table.json: for every (shape, activation rows, w_bits) of the benchmark configurations,
the kernel and launch geometry that ap_matmul_kbit picks under the default knobs, the routes of the q/k/v and gate/up
sets through ap_matmul_kbit_group, and whether the fused GEMM is taken at the batch sizes the module sees.

    python tests/golden/make_routing_table.py

The table is a record of the shipped launch rules (fitted to measurements on MI355X), not of a reference behaviour:
tests/test_routing_table.py fails when a rule edit moves any of these shapes, so that such a move is deliberate --
re-run this script and commit the new table together with the measurement that justifies it.  No GPU is needed: the
queries only evaluate the rules (256 compute units are assumed when no device is present).
"""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.join(ROOT, "any-precision-llm_amd"))

from any_precision_amd import _capi, synth  # noqa: E402

BITS = range(3, 9)


def build_table() -> dict:
    single, sets, fused = {}, {}, {}
    shapes_7b = sorted({(N, K) for _, N, K in synth.LLAMA2_7B_LAYER})
    shapes_8b = sorted({(N, K) for _, N, K in synth.LLAMA3_8B_LAYER})
    for N, K in shapes_7b:                       # configurations 1 and 2: batch 1
        for b in BITS:
            geo = _capi.matmul_geometry(1, N, K, b)
            single[f"{N}x{K}:M1:b{b}"] = [_capi.matmul_route(1, N, K, b), geo["rows"], geo["wpl"]]
    for N, K in shapes_8b:                       # configuration 3: batches 1, 2, 4, 8
        for M in (1, 2, 4, 8):
            for b in BITS:
                geo = _capi.matmul_geometry(M, N, K, b)
                single[f"{N}x{K}:M{M}:b{b}"] = [_capi.matmul_route(M, N, K, b), geo["rows"], geo["wpl"]]
    for name, rows, K in (("7b_qkv", [4096] * 3, 4096), ("7b_gate_up", [11008] * 2, 4096),
                          ("8b_qkv", [4096, 1024, 1024], 4096), ("8b_gate_up", [14336] * 2, 4096)):
        for M in (1, 2, 4, 8):
            for b in BITS:
                routes, per_wg = _capi.matmul_group_route(M, rows, K, b)
                sets[f"{name}:M{M}:b{b}"] = [routes, per_wg]
    for N, K in shapes_7b:                       # configuration 5: prompt (128 rows) and prefill (16384 rows), and between
        for M in (16, 128, 512, 16384):
            for b in BITS:
                fused[f"{N}x{K}:M{M}:b{b}"] = _capi.gemm_pays(M, N, K, b)
    for M in (16, 128, 512):
        for b in BITS:
            fused[f"7b_qkv_set:M{M}:b{b}"] = _capi.gemm_group_pays(M, [4096] * 3, 4096, b)
            fused[f"7b_gate_up_set:M{M}:b{b}"] = _capi.gemm_group_pays(M, [11008] * 2, 4096, b)
    return {"matmul_kbit": single, "matmul_kbit_group": sets, "fused_gemm_pays": fused}


if __name__ == "__main__":
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "routing_table.json")
    with open(out, "w") as f:
        json.dump(build_table(), f, indent=0, sort_keys=True)
        f.write("\n")
    print("wrote", out)
