"""Build recipe for libelectrock_moe.so (gfx950 only).

The library is compiled in-tree with plain hipcc; there is no CPU build of the
kernels and no fallback: importing the ops without the built library fails.

The tiled GEMM kernels copy global memory straight into LDS from inline assembly
and count the copies in flight by hand (csrc/lds_copy.h).  That accounting holds
only while the compiler adds no memory operations of its own to those kernels, so
the build checks what the compiler reports about them (its resource-usage remarks:
no scratch memory, no spilled vector registers, registers within one wave's share
of a SIMD at two waves per SIMD) and that the compiler is the release the kernels
were validated with.  A change of either fails the build here, on the CPU, instead
of showing up as wrong results on a GPU.
"""
import glob
import os
import re
import shutil
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libelectrock_moe.so")

HIPCC_FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-shared",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    # one block of remarks per kernel: registers, scratch, spills, LDS (read back by check_kernel_resources)
    "-Rpass-analysis=kernel-resource-usage",
]

# The compiler release the hand-scheduled kernels were validated with (`hipcc --version`).
VALIDATED_HIP = "7.2.26015"
VALIDATED_CLANG = "roc-7.2.0"

# Kernels whose copy pipelines are hand-counted: name fragment -> limits on the compiler's report.
# 512 threads = two waves per SIMD, so a wave owns 256 of the 512 registers of a SIMD lane; the 256-row kernel
# takes its 160 KB of LDS dynamically (reported as 0 static bytes), the streaming kernel (no hand-counted copies,
# two workgroups of four waves per CU) declares 36 KB.
GUARDED_KERNELS = {
    "gemm_tile_kernel": {"max_vgprs": 256, "min_vgprs": 200, "lds": 0},
    "gemm_tile_mid_kernel": {"max_vgprs": 256, "min_vgprs": 100, "lds": 0},
    "gemm_stream_kernel": {"max_vgprs": 256, "min_vgprs": 100, "lds": 36864},
}


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; libelectrock_moe.so cannot be built")


def sources():
    return sorted(glob.glob(os.path.join(CSRC_DIR, "*.hip")))


def check_compiler(hipcc: str) -> str:
    """The version text of hipcc; raises when it is not the validated release (set ELECTROCK_ALLOW_ANY_HIPCC=1 to
    build anyway, after checking the copy pipelines of csrc/lds_copy.h against the new compiler's code)."""
    text = subprocess.run([hipcc, "--version"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True).stdout
    ok = VALIDATED_HIP in text and VALIDATED_CLANG in text
    if not ok and os.environ.get("ELECTROCK_ALLOW_ANY_HIPCC") != "1":
        raise RuntimeError(
            f"hipcc is not the validated release (HIP {VALIDATED_HIP}, clang {VALIDATED_CLANG}):\n{text}\n"
            "the tiled GEMM kernels count their global->LDS copies by hand (csrc/lds_copy.h); re-validate them with "
            "this compiler (GPU tests, kernel resource report) and update VALIDATED_* in _build.py, or set "
            "ELECTROCK_ALLOW_ANY_HIPCC=1")
    return text


def parse_kernel_resources(log: str) -> dict:
    """{kernel name: {"sgprs", "vgprs", "agprs", "scratch", "sgpr_spill", "vgpr_spill", "lds"}} from the compiler's
    -Rpass-analysis=kernel-resource-usage remarks."""
    keys = {"TotalSGPRs": "sgprs", "VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch",
            "SGPRs Spill": "sgpr_spill", "VGPRs Spill": "vgpr_spill", "LDS Size [bytes/block]": "lds"}
    out, cur = {}, None
    for line in log.splitlines():
        m = re.search(r"remark: (?:\s*)Function Name: (\S+)", line)
        if m:
            cur = out.setdefault(m.group(1), {})
            continue
        m = re.search(r"remark:\s+([A-Za-z \[\]/]+): (\d+)", line)
        if m and cur is not None and m.group(1).strip() in keys:
            cur[keys[m.group(1).strip()]] = int(m.group(2))
    return out


def check_kernel_resources(resources: dict) -> list:
    """Raise if a guarded kernel uses scratch memory, spills vector registers or leaves its register / LDS bounds;
    returns the checked (name, report) pairs."""
    checked, problems = [], []
    for name, rep in sorted(resources.items()):
        for frag, lim in GUARDED_KERNELS.items():
            # mangled names hold the length-prefixed identifier, e.g. 16gemm_tile_kernel
            if f"{len(frag)}{frag}" not in name:
                continue
            checked.append((name, rep))
            if rep.get("scratch", 0) != 0 or rep.get("vgpr_spill", 0) != 0:
                problems.append(f"{name}: scratch {rep.get('scratch')} B/lane, {rep.get('vgpr_spill')} spilled VGPRs")
            if not lim["min_vgprs"] <= rep.get("vgprs", -1) + rep.get("agprs", 0) <= lim["max_vgprs"]:
                problems.append(f"{name}: {rep.get('vgprs')} VGPRs + {rep.get('agprs')} AGPRs outside "
                                f"[{lim['min_vgprs']}, {lim['max_vgprs']}]")
            if rep.get("lds", -1) != lim["lds"]:
                problems.append(f"{name}: {rep.get('lds')} B of static LDS, expected {lim['lds']}")
    found = {frag for frag in GUARDED_KERNELS if any(f"{len(frag)}{frag}" in n for n, _ in checked)}
    for frag in GUARDED_KERNELS:
        if frag not in found:
            problems.append(f"no resource report for any {frag}: the build no longer emits the remarks")
    if problems:
        raise RuntimeError("kernel resource check failed (the hand-counted copy pipelines need kernels without "
                           "compiler-made memory traffic):\n  " + "\n  ".join(problems))
    return checked


def build(verbose: bool = False) -> str:
    """Compile every HIP source into lib/libelectrock_moe.so; returns its path."""
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = hipcc_path()
    check_compiler(hipcc)
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc, *HIPCC_FLAGS, *sources(), "-o", tmp]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass prints one harmless line per file about the packed-fp32 feature
    lines = [l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l]
    # everything but the resource remarks (each is three lines: the remark, the source line, a caret)
    log, skip = [], 0
    for l in lines:
        if "[-Rpass-analysis=kernel-resource-usage]" in l:
            skip = 2
            continue
        if skip and (re.match(r"^\s*\d+ \|", l) or re.match(r"^\s*\|\s*\^", l)):
            skip -= 1
            continue
        skip = 0
        log.append(l)
    log = "\n".join(log)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + log)
    checked = check_kernel_resources(parse_kernel_resources(proc.stdout))
    if verbose:
        if log.strip():
            print(log)
        for name, rep in checked:
            print(f"{name}: {rep}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
