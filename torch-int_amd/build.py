"""Builds libtorch_int_hip.so (gfx950) in-tree with hipcc.

Run as a script (``python torch-int_amd/build.py``) or call ``build()``.
The library lands in ``torch-int_amd/torch_int/lib/`` next to the Python
package that loads it with ctypes.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "torch_int", "lib")
LIB_PATH = os.path.join(LIB_DIR, "libtorch_int_hip.so")
# (source, extra defines, object name).  The GEMM kernels are compiled once per epilogue kind (EpiKind 0..8 of
# csrc/ti_common.h), each kind in a translation unit of its own, so that they build in parallel.
SOURCES = [(s, [], s[:-4] + ".o") for s in
           ["api.hip", "gemm_s8.hip", "ln_q.hip", "softmax_q.hip", "permute.hip", "bmm_rowmajor.hip", "decode_attn.hip",
            "attn_fused.hip", "attn_long.hip", "diag_mfma.hip"]]
SOURCES += [("gemm_s8_kinds.hip", [f"-DTI_KIND={k}"], f"gemm_s8_kind{k}.o") for k in range(9)]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-ffp-contract=off",              # the epilogues spell out every fma themselves
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def build_fastcall(verbose=True):
    """The optional CPython forwarder (plain C, gcc): cuts per-call overhead of the Python wrappers."""
    import sysconfig
    out = os.path.join(LIB_DIR, "_ti_fastcall" + sysconfig.get_config_var("EXT_SUFFIX"))
    cmd = ["gcc", "-O2", "-fPIC", "-shared", "-Wall", "-I" + sysconfig.get_paths()["include"],
           os.path.join(CSRC, "fastcall.c"), "-o", out, "-L" + LIB_DIR, "-ltorch_int_hip", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return out


def write_kernel_resources(remarks):
    """The compiler's per-kernel resource remarks as torch_int/lib/kernel_resources.json: registers, scratch bytes per
    lane (register spills) and occupancy of every kernel in the library.  A kernel that starts to spill after an edit
    still computes the right bits, only several times slower; tests/test_abi.py reads this file."""
    import json
    import re
    kernels, name = {}, None
    for ln in remarks:
        m = re.search(r"remark: (?:[^:]*:\d+:\d+: )?(.*?) \[-Rpass-analysis", ln)
        text = m.group(1).strip() if m else ln
        if text.startswith("Function Name:"):
            name = text.split(":", 1)[1].strip()
            kernels[name] = {}
        elif name is not None:
            for key, label in (("vgprs", "VGPRs:"), ("agprs", "AGPRs:"), ("scratch_bytes_per_lane", "ScratchSize [bytes/lane]:"),
                               ("occupancy_waves_per_simd", "Occupancy [waves/SIMD]:"), ("lds_bytes_per_block", "LDS Size [bytes/block]:")):
                if text.startswith(label):
                    kernels[name][key] = int(text.split(":", 1)[1].strip())
    with open(os.path.join(LIB_DIR, "kernel_resources.json"), "w") as f:
        json.dump({"kernels": kernels}, f, indent=0, sort_keys=True)
    return kernels


def build(verbose=True, extra_flags=()):
    """Compiles every source to an object file (in parallel: the files are independent) and links them."""
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)

    def compile_one(item):
        src, defines, name = item
        obj = os.path.join(obj_dir, name)
        cmd = [HIPCC, *FLAGS, "-Rpass-analysis=kernel-resource-usage", *defines, *extra_flags, "-c",
               os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        done = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
        remarks = [ln for ln in done.stderr.splitlines() if "[-Rpass-analysis=kernel-resource-usage]" in ln]
        rest = [ln for ln in done.stderr.splitlines() if "[-Rpass-analysis=kernel-resource-usage]" not in ln]
        if verbose or done.returncode:
            sys.stdout.write(done.stdout)
            sys.stderr.write("\n".join(rest) + ("\n" if rest else ""))
        if done.returncode:
            raise subprocess.CalledProcessError(done.returncode, cmd)
        return obj, remarks

    with ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 4, 16)) as pool:
        results = list(pool.map(compile_one, SOURCES))
    objs = [obj for obj, _ in results]
    write_kernel_resources([ln for _, remarks in results for ln in remarks])
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    build_fastcall(verbose)
    return LIB_PATH


if __name__ == "__main__":
    build(extra_flags=sys.argv[1:])
