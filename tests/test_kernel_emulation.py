"""The few-row GEMM kernels' own source text (the 4-bit one, the e4m3 one and the general one), compiled for the host and run thread for thread on the CPU
(tests/kernel_emu/emu.h stands in for workgroups, waves, LDS, shuffles and the matrix instruction) under the
launch plans the library itself works out, with AddressSanitizer and UBSan: results against a plain fp64
product, every result element written, and no access outside the operands, the planes or the LDS.  What this
cannot show is the compiler's and the hardware's side (covered by the GPU tests); what it does show is the
kernel's indexing, its arithmetic identities and the host/kernel contract for shapes and row counts at will."""
import concurrent.futures
import json
import os
import re
import shutil
import subprocess
import sys

import pytest

from rustane_amd import hipdec
from rustane_amd.hipdec import WeightDtype

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EMU = os.path.join(ROOT, "tests", "kernel_emu")


def host_clang():
    for c in ("/opt/rocm/lib/llvm/bin/clang++", shutil.which("amdclang++"), shutil.which("clang++")):
        if c and os.path.exists(c):
            return c
    return None


@pytest.fixture(scope="module")
def emulator(tmp_path_factory):
    cxx = host_clang()
    if cxx is None:
        pytest.skip("no clang++ for the host (the kernel text uses clang's vector types)")
    build = tmp_path_factory.mktemp("kernel_emu")
    text = open(os.path.join(ROOT, "rustane_amd", "csrc", "hipdec_prefill.h")).read()
    start, end = text.index("#define PF_SQ_GU"), text.index("// The same few-row GEMM for e4m3 weights.")
    kernel = text[start:end]
    assert "void k_pf_gemm_skinny_i4(PfGemm g)" in kernel
    lds_decl = "extern __shared__ __align__(16) uint16_t s_act[];"
    assert kernel.count(lds_decl) == 1
    (build / "kernel_i4.inc").write_text(kernel.replace(lds_decl, "uint16_t *s_act = emu::lds();"))
    (build / "pfgemm_struct.inc").write_text(re.search(r"struct PfGemm \{.*?\n\};\n", text, flags=re.S).group(0))
    start, end = text.index("#define PF_S8_GU"), text.index("// ---------------------------------------------------------------- causal attention over the chunk")
    kernel = text[start:end]
    assert "void k_pf_gemm_skinny_f8(PfGemm g)" in kernel and kernel.count(lds_decl) == 1
    (build / "kernel_f8.inc").write_text(kernel.replace(lds_decl, "uint16_t *s_act = emu::lds();"))
    # the general kernel with the two helpers it calls (the pair split of fp32 weights)
    helpers = text[text.index("typedef __bf16 pf_bf16x2 __attribute__((ext_vector_type(2)));"):text.index("__device__ __forceinline__ float pf_block_sum(")]
    kernel = text[text.index("#define PF_SK_UNROLL 4"):text.index("// The few-row GEMM for 4-bit weights.  In k_pf_gemm_skinny")]
    assert "void k_pf_gemm_skinny(PfGemm g)" in kernel and kernel.count(lds_decl) == 1 and "pf_split2" in helpers
    (build / "kernel_few.inc").write_text(helpers + kernel.replace(lds_decl, "uint16_t *s_act = emu::lds();"))
    # the element-wise kernels between the products (with the helpers in front of them) and the multi-row step's two
    batch = open(os.path.join(ROOT, "rustane_amd", "csrc", "hipdec_batch.h")).read()
    epi = (text[text.index("// f16 != 0: the activation as ONE fp16 number in hi"):text.index("// ---------------------------------------------------------------- GEMM on the bf16 matrix cores")]
           + batch[batch.index("struct BatchParams {"):batch.index("// One workgroup per (head, row): online softmax over the shared prefix rows")]
           + batch[batch.index("// logits[r][v] = inv_rms[r] * sum_z P[z][r][v]"):batch.index("// ---- head kernels, one grid row per sequence")])
    for k in ("void k_pf_resid(", "void k_pf_gate_epi(", "void k_bd_qkv_epi(", "void k_bd_sum_planes(", "void pf_sum_planes("):
        assert k in epi, k
    (build / "kernels_epi.inc").write_text(epi)
    # the multi-row step's attention kernel with the cache-row decoders and the pair split it calls
    common = open(os.path.join(ROOT, "rustane_amd", "csrc", "hipdec_common.h")).read()
    att = (common[common.index("template <int WT> struct WS;"):common.index("template <> struct WS<WT_FP8> {")]
           + text[text.index("// f16 != 0: the activation as ONE fp16 number in hi"):text.index("typedef __bf16 pf_bf16x2 __attribute__((ext_vector_type(2)));")]
           + batch[batch.index("struct BatchParams {"):batch.index("// q/k/v rows of the step: sum the split planes")]
           + batch[batch.index("// One workgroup per (head, row): online softmax over the shared prefix rows"):batch.index("// logits[r][v] = inv_rms[r] * sum_z P[z][r][v]")])
    assert "void k_bd_attn(" in att and "struct WS<WT_BF16>" in att and "void pf_split(" in att
    (build / "kernel_bd_attn.inc").write_text(att)
    # the multi-row step's greedy and top-k head kernels with the ordering they share
    sel = (common[common.index("// (value desc, index asc) ordering used by every head kernel of the reference"):common.index("// 16-byte load of data that is used once per step")]
           + batch[batch.index("struct BatchParams {"):batch.index("// q/k/v rows of the step: sum the split planes")]
           + batch[batch.index("// ---- head kernels, one grid row per sequence"):batch.index("__global__ __launch_bounds__(256) void k_bd_block_stats(")])
    assert "void k_bd_argmax(" in sel and "void k_bd_topk(" in sel and "bool better(" in sel
    (build / "kernels_sel.inc").write_text(sel)
    # the weight conversion kernel with the e4m3 encoder; the oracle's C file is linked in as its checker
    kern = open(os.path.join(ROOT, "rustane_amd", "csrc", "hipdec_kernels.h")).read()
    enc = common[common.index("// software OCP e4m3fn encoder, round to nearest even, saturating"):]
    conv = (enc[:enc.index("\n}\n") + 3]
            + common[common.index("__device__ __forceinline__ float wave_max(float v) {"):common.index("// (value desc, index asc) ordering used by every head kernel of the reference")]
            + kern[kern.index("// one workgroup per source row of an out-major fp32 matrix [rows][K]; destination row ="):kern.index("// inverse of k_convert_rows for verification: stored row -> fp32")])
    assert "void k_convert_rows(" in conv and "uint8_t f32_to_e4m3(" in conv
    (build / "kernel_convert.inc").write_text(conv)
    # the single-row attention kernel of the one-kernel-per-product path
    ad = (common[common.index("struct StepParams {"):common.index("enum { WT_F32 = 0")]
          + common[common.index("template <int WT> struct WS;"):common.index("template <> struct WS<WT_FP8> {")]
          + kern[kern.index("// ---------------------------------------------------------------- attention (one query row)"):kern.index("// ---------------------------------------------------------------- heads (on the raw logits)")])
    assert "void k_attn_decode(" in ad
    (build / "kernel_attn_decode.inc").write_text(ad)
    # the matrix-vector kernel of the same path with the four weight decoders (shared with the persistent kernels); its
    # empty asm that pins a register names a GPU register class, and its LDS declaration becomes the stand-in's block
    gv = (common[common.index("struct StepParams {"):common.index("enum { WT_F32 = 0")]
          + common[common.index("template <int WT> struct WS;"):common.index("// software OCP e4m3fn encoder, round to nearest even, saturating")]
          + kern[kern.index("enum { EPI_QKV = 0"):kern.index("// ---------------------------------------------------------------- embedding / input")]
          + kern[kern.index("// ---------------------------------------------------------------- GEMV"):kern.index("// ---------------------------------------------------------------- attention (one query row)")])
    pin, xs_decl = 'asm volatile("" : "+v"(hi));', "extern __shared__ __align__(16) float xs[];"
    assert gv.count(pin) == 1 and gv.count(xs_decl) == 1 and "void k_gemv(GemvArgs a)" in gv
    (build / "kernel_gemv.inc").write_text(gv.replace(pin, 'asm volatile("" : "+r"(hi));').replace(xs_decl, "float *xs = (float *)emu::lds();"))
    # the top-k draw on the device with the restated host expf / tanhf and the run state
    smp = open(os.path.join(ROOT, "rustane_amd", "csrc", "hipdec_sample.h")).read()
    draw = (common[common.index("// (value desc, index asc) ordering used by every head kernel of the reference"):common.index("// 16-byte load of data that is used once per step")]
            + batch[batch.index("struct BatchParams {"):batch.index("// q/k/v rows of the step: sum the split planes")]
            + smp[smp.index("__host__ __device__ __forceinline__ uint64_t sample_exp2_tab(unsigned i) {"):smp.index("// order-independent checksum of a restated function")]
            + smp[smp.index("// ---------------------------------------------------------------- run state"):smp.index("// One workgroup per row: the block from the statistics, then the token inside the block.")])
    assert "void k_sample_topk(" in draw and "float expf_as_host(" in draw and "float tanhf_as_host(" in draw
    (build / "kernel_sample.inc").write_text(draw)
    # the full-vocabulary draw: block from the statistics, token inside the block
    softcap_line = "__device__ __forceinline__ float softcap_dev(float x, float cap) { return cap > 0.0f ? cap * tanhf(x / cap) : x; }\n"
    assert softcap_line in kern
    fv = smp[smp.index("// One workgroup per row: the block from the statistics, then the token inside the block."):]
    fv = (common[common.index("__device__ __forceinline__ float wave_max(float v) {"):common.index("// (value desc, index asc) ordering used by every head kernel of the reference")]
          + batch[batch.index("struct BatchParams {"):batch.index("// q/k/v rows of the step: sum the split planes")] + softcap_line
          + smp[smp.index("__host__ __device__ __forceinline__ uint64_t sample_exp2_tab(unsigned i) {"):smp.index("// order-independent checksum of a restated function")]
          + smp[smp.index("// ---------------------------------------------------------------- run state"):smp.index("// One workgroup per row.  vals/idxs: [rows][blocks * top_k]")]
          + "#define SAMPLE_MAX_BLOCKS 1024\n" + fv[:fv.index("\n}\n") + 3])
    assert "void k_sample_fullvocab(" in fv and "#define SAMPLE_MAX_BLOCKS 1024" in smp
    (build / "kernel_sample_fv.inc").write_text(fv)
    # the single-row head kernels and the multi-row block statistics
    bst = batch[batch.index("__global__ __launch_bounds__(256) void k_bd_block_stats("):]
    heads = (common[common.index("struct StepParams {"):common.index("enum { WT_F32 = 0")]
             + common[common.index("__device__ __forceinline__ float wave_max(float v) {"):common.index("// 16-byte load of data that is used once per step")]
             + kern[kern.index("// ---------------------------------------------------------------- heads (on the raw logits)"):kern.index("__global__ void k_advance(StepParams *sp)")]
             + batch[batch.index("struct BatchParams {"):batch.index("// q/k/v rows of the step: sum the split planes")] + bst[:bst.index("\n}\n") + 3])
    for k in ("void k_head_argmax(", "void k_head_topk(", "void k_head_block_stats(", "void k_softcap_copy(", "void k_bd_block_stats("):
        assert k in heads, k
    (build / "kernels_heads.inc").write_text(heads)
    # the tiled prefill GEMM with its helpers
    tiled = text[text.index("struct PfGemm {"):text.index("#define PF_DL_BM 128")]
    assert "void k_pf_gemm(PfGemm g)" in tiled
    (build / "kernel_tiled.inc").write_text(tiled)
    oracle_o = build / "oracle.o"
    r = subprocess.run([cxx.replace("clang++", "clang"), "-O1", "-w", "-c", os.path.join(ROOT, "oracle", "rustane_oracle.c"), "-o", str(oracle_o)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    exes = {}
    programs = (("epilogues", ["-Wno-psabi"]), ("batch_attention", ["-Wno-psabi"]), ("selection", []), ("single_row_attention", ["-Wno-psabi"]),
                ("gemv", ["-Wno-psabi"]), ("convert_rows", [str(oracle_o), "-lm"]),
                ("sample_topk", ["-ffp-contract=off", "-Wno-psabi", str(oracle_o), "-lm"]),
                ("sample_fullvocab", ["-ffp-contract=off", "-Wno-psabi", str(oracle_o), "-lm"]),
                ("single_row_heads", ["-ffp-contract=off", "-Wno-psabi", str(oracle_o), "-lm"]), ("tiled_gemm", ["-Wno-psabi"]), ("few_row_i4", []),
                ("few_row_f8", ["-DEMU_F8_WAVES=8", "-DEMU_F8_KERNEL(RT,PACK)=k_pf_gemm_skinny_f8<RT,PACK,8>"]), ("few_row_general", ["-Wno-psabi"]))

    def compile_one(item):
        name, extra = item
        cmd = [cxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer",
               "-pthread", *extra, "-I", str(build), "-I", EMU, os.path.join(EMU, name + ".cpp"), "-o", str(build / name)]
        return name, subprocess.run(cmd, capture_output=True, text=True)

    with concurrent.futures.ThreadPoolExecutor(max_workers=4) as pool:
        for name, r in pool.map(compile_one, programs):
            assert r.returncode == 0, (name, r.stderr[-4000:])
            exes[name] = str(build / name)
    return exes


def run_case(exes, wd, rows, n, k, num_cu, seed, lds_delta=0):
    p = hipdec.gemm_plan(wd, rows, n, k, num_cu)
    assert p["kernel"] == ("few_row_int4" if wd == WeightDtype.INT4_G128 else "few_row_e4m3")
    exe = exes["few_row_i4" if wd == WeightDtype.INT4_G128 else "few_row_f8"]
    args = [rows, n, k, p["steps_per_split"], *p["grid"], p["threads"], p["lds_bytes"] + lds_delta, seed]
    r = subprocess.run([exe] + [str(a) for a in args], capture_output=True, text=True, timeout=600)
    return p, r


# (rows, n, k, compute units the plan is made for): packed hi/lo tile up to 8 rows, one and two row tiles above;
# reductions of 1, 3, 5, 9 and 16 scale groups; ragged n; splits of 1, 2, 3, 4 and 8 groups (the last through plans
# for a small device, which keep the grid small enough to emulate)
CASES = [
    (8, 300, 384, 256), (5, 130, 1152, 256), (1, 16, 128, 256), (3, 257, 640, 256), (8, 128, 2048, 256),
    (8, 512, 2048, 2), (7, 384, 1024, 1), (16, 200, 640, 256), (9, 129, 384, 256), (13, 256, 2048, 2),
    (27, 70, 384, 256), (17, 130, 1152, 256), (32, 144, 640, 256), (32, 256, 1024, 1),
]


@pytest.mark.parametrize("rows,n,k,num_cu", CASES)
def test_four_bit_few_row_kernel_source_on_the_cpu(emulator, rows, n, k, num_cu):
    p, r = run_case(emulator, WeightDtype.INT4_G128, rows, n, k, num_cu, seed=rows * 1000 + n)
    assert r.returncode == 0, (p, r.stdout, r.stderr[-3000:])
    assert "not written 0" in r.stdout


# e4m3: reductions of 1 to 32 blocks of 64 elements (k need not be a multiple of 128), splits of 1 to 8 blocks
CASES_E4M3 = [
    (8, 300, 384, 256), (5, 130, 1152, 256), (1, 16, 64, 256), (3, 257, 704, 256), (8, 256, 2048, 2), (7, 384, 1024, 1),
    (16, 200, 640, 256), (9, 129, 448, 256), (19, 160, 1024, 256), (20, 160, 1024, 256), (27, 70, 384, 256), (32, 144, 640, 256),
]


@pytest.mark.parametrize("rows,n,k,num_cu", CASES_E4M3)
def test_e4m3_few_row_kernel_source_on_the_cpu(emulator, rows, n, k, num_cu):
    p, r = run_case(emulator, WeightDtype.FP8_E4M3, rows, n, k, num_cu, seed=rows * 1000 + n)
    assert r.returncode == 0, (p, r.stdout, r.stderr[-3000:])
    assert "not written 0" in r.stdout


@pytest.mark.parametrize("wd", [WeightDtype.INT4_G128, WeightDtype.FP8_E4M3])
def test_the_sanitizer_sees_an_access_past_the_lds(emulator, wd):
    # the control for the tests above: with less LDS than the staged rows take, the same launch is reported
    p, r = run_case(emulator, wd, 8, 300, 384, 256, 1, lds_delta=-640)
    assert r.returncode != 0 and "heap-buffer-overflow" in r.stderr, (p, r.stdout, r.stderr[-2000:])


# the general few-row kernel: all four weight formats (fp32 weights as bf16 pairs, bf16, e4m3 widened in registers,
# 4-bit through the integer trick); the library plans it for e4m3 and 4-bit weights only with the kernels of their
# own switched off, which the environment decides once per process -- so these plans come from a child process
CASES_GENERAL = [(8, 100, 384, 256), (5, 130, 1152, 256), (16, 65, 640, 256), (27, 70, 384, 256), (32, 64, 1024, 2), (1, 33, 128, 256)]


@pytest.fixture(scope="module")
def general_plans():
    code = ("import json; from rustane_amd import hipdec; "
            "print(json.dumps([[wd, c, hipdec.gemm_plan(wd, *c)] for wd in range(4) for c in %r if not (wd == 3 and c[2] %% 128)]))" % (CASES_GENERAL,))
    env = dict(os.environ, HIPDEC_NO_SKINNY_I4="1", HIPDEC_NO_SKINNY_F8="1")
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=ROOT, env=env, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    return json.loads(r.stdout)


def test_general_few_row_kernel_source_on_the_cpu(emulator, general_plans):
    assert len(general_plans) == 4 * len(CASES_GENERAL)
    for wd, (rows, n, k, num_cu), p in general_plans:
        assert p["kernel"] == "few_row", (wd, p)
        args = [wd, rows, n, k, p["steps_per_split"], *p["grid"], p["threads"], p["lds_bytes"], rows * 1000 + n]
        r = subprocess.run([emulator["few_row_general"]] + [str(a) for a in args], capture_output=True, text=True, timeout=600)
        assert r.returncode == 0 and "not written 0" in r.stdout, (wd, p, r.stdout, r.stderr[-3000:])


def test_element_wise_kernels_source_on_the_cpu(emulator):
    # k_pf_embed, k_pf_qkv_epi, k_pf_resid, k_pf_gate_epi, k_bd_qkv_epi (both cache formats) and k_bd_sum_planes against fp64 restatements, with
    # split counts on both sides of the plane sums' request rounds of four and eight
    r = subprocess.run([emulator["epilogues"]], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0 and "0 checks failed" in r.stdout, (r.stdout[-4000:], r.stderr[-3000:])
    assert r.stdout.count("k_pf_resid") >= 11 and r.stdout.count("k_bd_qkv_epi") >= 6
    assert r.stdout.count("k_pf_embed<") == 2 and r.stdout.count("k_pf_qkv_epi<") == 6


def test_multi_row_attention_kernel_source_on_the_cpu(emulator):
    # k_bd_attn (1024 threads per (head, row)) against an fp64 softmax attention over prefix + suffix rows: both cache
    # formats, head dimensions 64 and 128, grouped heads, row counts below one pass, inside a pass and over several
    r = subprocess.run([emulator["batch_attention"]], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0 and "0 checks failed" in r.stdout, (r.stdout[-4000:], r.stderr[-3000:])
    assert r.stdout.count("k_bd_attn<") == 6


def test_greedy_and_top_k_head_kernels_source_on_the_cpu(emulator):
    # k_bd_argmax and k_bd_topk against a sort by (value descending, index ascending): ties, -inf entries, a block of
    # nothing but -inf, vocabularies that end inside a block, k above the number of rows (padded lists)
    r = subprocess.run([emulator["selection"]], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0 and "0 checks failed" in r.stdout, (r.stdout[-4000:], r.stderr[-3000:])
    assert r.stdout.count("0 mismatches") == 5


def test_weight_conversion_kernel_source_on_the_cpu(emulator):
    # k_convert_rows: stored e4m3 rows + row scales and stored 4-bit rows + bf16 group scales bit for bit against the
    # oracle's quantisers, bf16 rows to the nearest, with the interleaving row map
    r = subprocess.run([emulator["convert_rows"]], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0 and "0 checks failed" in r.stdout, (r.stdout[-4000:], r.stderr[-3000:])
    assert r.stdout.count("0 mismatches") == 4


def test_single_row_attention_kernel_source_on_the_cpu(emulator):
    # k_attn_decode ((head, split) workgroups, the last of a head folds the partial records) against an fp64 softmax
    # attention: both cache formats, head dimensions 64 and 128, grouped heads, splits with few or no rows
    r = subprocess.run([emulator["single_row_attention"]], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0 and "0 checks failed" in r.stdout, (r.stdout[-4000:], r.stderr[-3000:])
    assert r.stdout.count("k_attn_decode<") == 5


def test_matrix_vector_kernel_source_on_the_cpu(emulator):
    # k_gemv for fp32, bf16, e4m3 and 4-bit weights with every fused prologue / epilogue (RMSNorm in; RoPE + cache
    # append with both cache formats, residual, both activations, logits out) against fp64 restatements
    r = subprocess.run([emulator["gemv"]], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0 and "0 checks failed" in r.stdout, (r.stdout[-4000:], r.stderr[-3000:])
    assert r.stdout.count("k_gemv<format") == 28


def test_top_k_draw_kernel_source_on_the_cpu(emulator):
    # k_sample_topk (candidate merge, softcap, softmax draw, LCG, run state) against the oracle's restatement of the
    # reference's host code, token for token and RNG state for RNG state over consecutive steps of several rows
    r = subprocess.run([emulator["sample_topk"]], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0 and "0 checks failed" in r.stdout, (r.stdout[-4000:], r.stderr[-3000:])
    assert r.stdout.count("0 mismatches") == 5


def test_full_vocabulary_draw_kernel_source_on_the_cpu(emulator):
    # k_sample_fullvocab (block from the statistics, then the token inside the block; two draws per token) against the
    # oracle's restatement of the reference's host code, token for token and RNG state for RNG state, with blocks of
    # nothing but -inf, softcap, a last block that is not full and more blocks than threads
    r = subprocess.run([emulator["sample_fullvocab"]], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0 and "0 checks failed" in r.stdout, (r.stdout[-4000:], r.stderr[-3000:])
    assert r.stdout.count("0 mismatches") == 4


def test_single_row_head_kernels_source_on_the_cpu(emulator):
    # k_head_argmax (with the step state it advances), k_head_topk (exact lists), k_head_block_stats / k_bd_block_stats
    # (exact maxima, sums at 1e-5) and k_softcap_copy against the oracle's restatements
    r = subprocess.run([emulator["single_row_heads"]], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0 and "0 checks failed" in r.stdout, (r.stdout[-4000:], r.stderr[-3000:])
    assert r.stdout.count("0 mismatches") == 4


# the tiled prefill GEMM: 33 rows up, two row tiles, ragged n, a reduction that ends inside a 64-element step
CASES_TILED = [(100, 200, 512, 256), (40, 130, 384, 4), (150, 257, 640, 256), (33, 64, 416, 256), (130, 140, 288, 256)]


@pytest.mark.parametrize("wd", [WeightDtype.BF16, WeightDtype.FP8_E4M3, WeightDtype.INT4_G128])
def test_tiled_prefill_gemm_kernel_source_on_the_cpu(emulator, wd):
    # k_pf_gemm for bf16, e4m3 and 4-bit weights with the three activation formats (bf16 pair, bf16 hi part, fp16)
    # under the library's plans against an fp64 product of the stored operands
    ran = 0
    for rows, n, k, num_cu in CASES_TILED:
        if wd == WeightDtype.INT4_G128 and k % 128:
            continue
        p = hipdec.gemm_plan(wd, rows, n, k, num_cu)
        if wd == WeightDtype.BF16 and rows >= 129 and k % 64 == 0:
            assert p["kernel"] == "tiled_direct_lds"       # (that kernel's loads write LDS directly: not emulated)
            continue
        assert p["kernel"] == "tiled" and p["threads"] == 256 and p["lds_bytes"] == 0, p
        for act in (0, 1, 2):
            args = [int(wd), act, rows, n, k, p["steps_per_split"], *p["grid"], rows + act]
            r = subprocess.run([emulator["tiled_gemm"]] + [str(a) for a in args], capture_output=True, text=True, timeout=600)
            assert r.returncode == 0 and "not written 0" in r.stdout, (wd, act, p, r.stdout, r.stderr[-3000:])
            ran += 1
    assert ran >= 6
