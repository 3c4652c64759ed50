#!/usr/bin/env python3
"""Registers, LDS, scratch and instruction mix of this library's own gfx950 kernels, read from the assembly that
hipcc emits for the sources in this directory (the device pass of `hipcc -S`, same flags as the Makefile).

usage: python3 dynet_amd/csrc/isa_mix.py [substring of a kernel name ...]      (no argument: the hot kernels)

Per kernel: VGPRs, AGPRs, SGPRs, bytes of LDS and of scratch from the kernel's metadata, and how many instructions of
each kind its body holds: 128-bit / narrower global loads and stores, loads straight into LDS, LDS accesses, DPP
row operations, cross-lane permutes and read-lanes, matrix-core instructions, and atomics on global memory (by type).
Counts are static (instructions in the code, not executed)."""
import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
SRCS = ["elementwise", "cwise", "reduce", "softmax", "lookup", "gemm", "gemm_wide", "gemm_small", "lstm", "misc", "trainer", "random"]
FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-function", "-Wno-unknown-warning-option", "-I" + os.path.join(HERE, "../../include"),
         "-I" + HERE, "--cuda-device-only", "-S"]
HOT = ["ew_vec4_kernel<2, true, 0, true, 2, dyhip::AccMul2", "ew_vec4_kernel<1, false, 0, true, 4, dyhip::TanhFwd",
       "ew_bcast_vec4_kernel<1, true, 1, true, 4, dyhip::AccIn0", "batch_reduce_kernel<4, false, true>",
       "ln_fwd_wave_kernel<4, true>", "ln_bwd_wave_kernel<4, true, 8, true, true>", "ln_bwd_team_kernel<4, true>",
       "combine_partials_vec_kernel<64>", "cwise_bcast2_kernel<2, 4, true>", "cwise_reduce_row_kernel<6, true, true>",
       "lookup_gather_kernel<HIP_vector_type<float, 4u>, false, true>", "plan_direct_kernel<16>", "plan_group_kernel<true>",
       "scatter_runs_kernel<HIP_vector_type<float, 4u>, true>", "lse_cols_kernel<true, true>", "pnls_bwd_kernel<true, true, true>",
       "lstm_step_fwd_kernel<false, 2>", "lstm_step_bwd_kernel", "skinny_tn_kernel<true, true>", "skinny_nn_kernel<2, 0, 16>", "skinny_nn_kernel<1, 1, 16>", "gemm_tn_mid_kernel<5>",
       "gemm_wide_kernel<false, false>", "gemm_shallow_nt_kernel", "gemm_tile_kernel<false, false, 1, 2>",
       "gather_segments_kernel<true, true>", "sgd_scaled_kernel<true, true>", "philox",
       "gemm_nn_mid_kernel<true>", "gemm_nn_rows_kernel<1, 8, 4>", "gemm_nn_thin_kernel<1>", "gemm_nt_thin_kernel<32, 4>",
       "gemm_tn_thin_kernel<4, 2>", "ln_fwd_group_kernel<16, 1, 2, true>", "ln_bwd_group_kernel<16, 1, true>",
       "sum_group_kernel<false, false>", "gemm_small_kernel<4, 4, 4>", "gemm_small_kernel<1, 4, 8>", "gemm_nt_fewrows_kernel<20>", "col_chunk_kernel<0>",
       "radix_scatter_kernel<true>", "radix_scan_kernel", "moment_chunk_kernel<1>", "rows_slab_kernel<false>",
       "batch_reduce_flat_kernel<false>", "pick_range_flat_kernel<false>", "softmax_resident_kernel<0, 256, 4>", "moment_resident_kernel<1, 256, 4>"]

KINDS = [
    ("ld128", r"^\s*(global|flat|buffer)_load_dwordx4\b"),
    ("ld<128", r"^\s*(global|flat|buffer)_load_(dword|dwordx2|dwordx3|ubyte|ushort|sbyte|sshort)\b"),
    ("ld->lds", r"^\s*(global|buffer)_load_lds_"),
    ("st128", r"^\s*(global|flat|buffer)_store_dwordx4\b"),
    ("st<128", r"^\s*(global|flat|buffer)_store_(dword|dwordx2|dwordx3|byte|short)\b"),
    ("lds", r"^\s*ds_(read|write|load|store)"),
    ("dpp", r"\b(row_shr|row_shl|row_ror|row_bcast|row_mirror|row_half_mirror|quad_perm|row_newbcast|row_share)"),
    ("permute", r"^\s*(ds_bpermute|ds_permute|ds_swizzle|v_permlane|v_readlane|v_readfirstlane|v_writelane)"),
    ("mfma", r"^\s*v_mfma_"),
    ("atomic_f", r"^\s*(global|flat|buffer)_atomic_(add_f|pk_add|fadd|fmin|fmax)"),
    ("atomic_i", r"^\s*(global|flat|buffer)_atomic_(?!add_f|pk_add|fadd|fmin|fmax)"),
    ("scratch", r"^\s*scratch_(load|store)"),
]


def demangle(names):
    out = subprocess.run(["c++filt"], input="\n".join(names), capture_output=True, text=True)
    return out.stdout.splitlines()


def kernels_of(asm):
    """{mangled name: (metadata dict, counts dict)} of one assembly file."""
    meta = {}
    for m in re.finditer(r"- \.agpr_count:.*?(?=\n  - \.agpr_count:|\namdhsa\.target|\n\.\.\.)", asm, re.S):
        blk = m.group(0)
        name = re.search(r"\.name:\s+(\S+)", blk).group(1)
        get = lambda k: int(re.search(r"\.%s:\s+(\d+)" % k, blk).group(1))
        meta[name] = {"vgpr": get("vgpr_count"), "agpr": get("agpr_count"), "sgpr": get("sgpr_count"),
                      "lds": get("group_segment_fixed_size"), "scratch": get("private_segment_fixed_size")}
    res = {}
    for name, md in meta.items():
        # the body: from the kernel's label to the function's end label (a kernel may hold several s_endpgm)
        m = re.search(r"^%s:[^\n]*\n(.*?)^\.Lfunc_end" % re.escape(name), asm, re.S | re.M)
        body = m.group(1) if m else ""
        counts = {k: 0 for k, _ in KINDS}
        for line in body.splitlines():
            for k, pat in KINDS:
                if re.search(pat, line):
                    counts[k] += 1
        res[name] = (md, counts)
    return res


def main():
    want = sys.argv[1:] or HOT
    rows = []
    with tempfile.TemporaryDirectory() as tmp:
        for src in SRCS:
            out = os.path.join(tmp, src + ".s")
            subprocess.run(["/opt/rocm/bin/hipcc"] + FLAGS + [os.path.join(HERE, src + ".hip"), "-o", out], check=True,
                           stderr=subprocess.DEVNULL)
            ks = kernels_of(open(out).read())
            names = list(ks)
            for mangled, plain in zip(names, demangle(names)):
                rows.append((src, plain, ks[mangled]))
    cols = ["vgpr", "agpr", "sgpr", "lds", "scratch"] + [k for k, _ in KINDS]
    print("%-92s %s" % ("kernel (file)", " ".join("%8s" % c for c in cols)))
    for w in want:
        for src, plain, (md, counts) in rows:
            if w in plain:
                short = re.sub(r"HIP_vector_type<float, 4u>", "float4", plain).replace("(anonymous namespace)::", "")
                short = re.sub(r"\(.*", "", short).replace("void ", "").replace("dyhip::", "").replace("(anonymous namespace)::", "")
                vals = [md[c] for c in cols[:5]] + [counts[c] for c in cols[5:]]
                print("%-92s %s" % ((short + " (" + src + ")")[:92], " ".join("%8d" % v for v in vals)))


if __name__ == "__main__":
    main()
