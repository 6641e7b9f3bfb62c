"""Builds libsglamd.so (the torch-free C-ABI library) for gfx950 with hipcc, in-tree.

Usage: python sglang_amd/csrc/build.py [-j N]   (run by path: importing the package needs the built library)
"""
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
LIB_PATH = os.path.join(PKG, "libsglamd.so")
SOURCES = ["gemm_mode_block_fp8.hip", "gemm_mode_row_fp8.hip", "gemm_mode_row_int8.hip", "gemm_mode_block_int8.hip",
           "moe.hip", "quant.hip", "gemm.hip", "generic.hip", "ceilings.hip"]
# packed fp32 ALU forms are switched off on purpose (the -Xclang -target-feature pair below)
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Wno-unused-result", "-Wno-unused-command-line-argument",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results feed v_fma directly in the block-scaled GEMMs: keep them in arch VGPRs
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    # one remark block per kernel with its registers, scratch and occupancy (parsed by _resource_table)
    "-Rpass-analysis=kernel-resource-usage",
]
# The GEMM kernels sit at the edge of the 256-VGPR budget their two waves per SIMD leave: a few more live values
# and the compiler spills accumulators into scratch memory, which still computes the right result, two to ten
# times slower.  A build in which a kernel of these files uses scratch memory therefore fails.
NO_SCRATCH = {"gemm_mode_block_fp8.hip", "gemm_mode_row_fp8.hip", "gemm_mode_row_int8.hip", "gemm_mode_block_int8.hip",
              "moe.hip"}


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _resource_table(stderr: str):
    """[(kernel, vgprs, agprs, sgprs, scratch bytes per lane, waves per SIMD)] from the compiler's remarks."""
    rows, seen = [], set()
    for block in stderr.split("Function Name: ")[1:]:
        name = block.split("\n", 1)[0].split(" [", 1)[0].strip()
        if name in seen:
            continue
        seen.add(name)

        def field(key):
            m = re.search(re.escape(key) + r": (\d+)", block)
            return int(m.group(1)) if m else -1

        rows.append((name, field("VGPRs"), field("AGPRs"), field("SGPRs"), field("ScratchSize [bytes/lane]"),
                     field("Occupancy [waves/SIMD]")))
    return rows


def _require_complete_report(src: str, table) -> None:
    """The scratch guard only means something when the compiler reported on every kernel: an empty table, or a
    kernel whose register or scratch field could not be read, fails the build instead of passing it unseen."""
    if not table:
        raise RuntimeError(f"{src}: the compiler printed no kernel-resource-usage remarks; the scratch guard "
                           "cannot be checked (did the remark format or the flag change?)")
    unread = [row[0] for row in table if row[1] < 0 or row[4] < 0]
    if unread:
        raise RuntimeError(f"{src}: no VGPR or scratch figure in the compiler's remarks for: " + ", ".join(unread))


def build(jobs: int = 4, verbose: bool = True) -> str:
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(HERE, s))]

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *HIPCC_FLAGS, "-c", os.path.join(HERE, src), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
        table = _resource_table(r.stderr)
        with open(os.path.join(objdir, src.replace(".hip", ".resources.txt")), "w") as f:
            f.write("kernel vgprs agprs sgprs scratch_bytes_per_lane waves_per_simd\n")
            for row in table:
                f.write(" ".join(str(v) for v in row) + "\n")
        spilling = [row for row in table if row[4] > 0]
        if src in NO_SCRATCH:
            _require_complete_report(src, table)
        if src in NO_SCRATCH and spilling:
            os.remove(obj)
            raise RuntimeError(f"{src}: kernels that must stay in registers use scratch memory: "
                               + ", ".join(f"{row[0]} ({row[4]} B/lane)" for row in spilling))
        return obj

    with ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        objs = list(ex.map(compile_one, srcs))
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} from {srcs}", file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    j = 4
    if "-j" in sys.argv:
        j = int(sys.argv[sys.argv.index("-j") + 1])
    build(jobs=j)
