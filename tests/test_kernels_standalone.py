"""Every kernel source compiles on its own with the command line the reference's kernel
cache uses (src/runtime/mod.rs:195-245: `hipcc --genco --offload-arch=<arch> -O3 -std=c++17
-I<dir> <file> -o <hsaco>`): the sources carry no dependence on a build system, and each file
exports the reference's symbol names.

This is a COMPILE-ONLY check (hipcc cross-compiles without a GPU); nothing built here is ever run.
The supported build -- the one every GPU test, the smoke and the benchmark load -- is the single
code object the Makefile in reinstinct_amd/csrc produces, with
`-Xclang -target-feature -Xclang -packed-fp32-ops -fhip-fp32-correctly-rounded-divide-sqrt`:
the first keeps the compiler from forming packed fp32 instructions, the second is part of the
bit-level definition of quantize_q8.  A host that compiles these files itself at run time must
pass the same flags; a code object built with the bare command above is untested."""
import concurrent.futures
import glob
import os
import shutil
import subprocess

import pytest

KDIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "reinstinct_amd", "csrc", "kernels")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"

# reference-named entry points a few of the files must export (names as the reference host looks them up)
EXPECT = {
    "quantize_q8.hip": [b"quantize_q8_f32"],
    "matvec_q4k_repacked.hip": [b"matvec_q4k_repacked_f32", b"matvec_q4k_repacked_r1_f32", b"matvec_q4k_repacked_r4_f32"],
    "matvec_q6k_repacked_batched.hip": [b"matvec_q6k_repacked_batched_f32", b"matvec_q6k_repacked_batched16_f32"],
    "mmq_gemm_q4k_repacked.hip": [b"mmq_gemm_q4k_repacked_f32", b"mmq_gemm_q4k_repacked_narrow_f32"],
    "mmq_gemm_q6k_grouped.hip": [b"mmq_gemm_q6k_grouped_f32"],
    "moe_expert_sort.hip": [b"moe_sort_zero", b"moe_sort_histogram", b"moe_sort_scan", b"moe_sort_scatter",
                            b"moe_gather_xq", b"moe_scatter_rows"],
    "moe_topk.hip": [b"moe_topk_f32"],
    "moe_combine.hip": [b"moe_combine_f32"],
    "swiglu.hip": [b"swiglu_mul_f32"],
}


def compile_one(src, out_dir):
    out = os.path.join(out_dir, os.path.basename(src) + ".hsaco")
    cmd = [HIPCC, "--genco", "--offload-arch=gfx950", "-O3", "-std=c++17", "-I" + KDIR, src, "-o", out]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    return src, out, p.returncode, p.stdout


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="no hipcc")
def test_each_kernel_file_compiles_alone_with_the_reference_command(tmp_path):
    files = sorted(f for f in glob.glob(os.path.join(KDIR, "*.hip")) if os.path.basename(f) != "rein_kernels.hip")
    assert len(files) >= 30
    with concurrent.futures.ThreadPoolExecutor(max_workers=8) as pool:
        results = list(pool.map(lambda f: compile_one(f, str(tmp_path)), files))
    failed = [(os.path.basename(s), log[-800:]) for s, _, rc, log in results if rc != 0]
    assert not failed, failed
    for src, out, _, _ in results:
        blob = open(out, "rb").read()
        for name in EXPECT.get(os.path.basename(src), []):
            assert name in blob, f"{os.path.basename(src)} does not export {name.decode()}"
