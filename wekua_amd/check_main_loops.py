"""Guard for the kernels that bring their k-slabs straight into LDS and count their own waits.

Their loads are issued from inline assembly, which the compiler's wait-count pass does not see; a wait of its
own that it puts into a main loop (s_waitcnt vmcnt(n) in front of a register it believes some earlier load may
still write) drains the slab pipeline in every iteration without changing any result -- a slow-down of 10-15 %
that no test notices.  This script compiles the files to assembly (device side only) and lists every loop block
that holds matrix instructions and direct-to-LDS loads together with a vmcnt wait that is not one of the
hand-written ones.  Run after changes to these kernels or to the compiler:

    python3 -m wekua_amd.check_main_loops          # exit status 1 when a loop has such a wait
"""
import os
import re
import subprocess
import sys
import tempfile

from . import build

FILES = [("wk_gemm_dma.hip", "gemm_f32_dma_kernel"), ("wk_gemm_dma_f64.hip", "gemm_f64_dma_kernel"),
         ("wk_gemm_ipack.hip", "gemm_i32_packed_dma_kernel"), ("wk_gemm_ipack.hip", "gemm_i8_packed_dma_kernel"),
         ("wk_gemm_ipack.hip", "gemm_i16_packed_dma_kernel"), ("wk_gemm_i64pack.hip", "gemm_i64_packed_kernel")]


def assembly(src: str, out: str) -> None:
    flags = [f for f in build.HIP_FLAGS if f != "-fPIC"]
    subprocess.run([build.HIPCC] + flags + ["--cuda-device-only", "-S", os.path.join(build.CSRC, src), "-o", out],
                   check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)


def scan(text: str, kernel: str):
    """[(mangled name tail, block label, [vmcnt values])] for the kernels whose name holds `kernel`."""
    found, kernels = [], 0
    parts = re.split(r"\n(_Z\w*" + kernel + r"\w*):\s", text)
    for i in range(1, len(parts), 2):
        kernels += 1
        body = parts[i + 1].split(".Lfunc_end")[0]
        for block in re.split(r"\n(?=\.LBB\d+_\d+:)", body):
            if block.count("v_mfma") >= 8 and "global_load_lds" in block:
                own = re.sub(r";;#ASMSTART.*?;;#ASMEND", "", block, flags=re.S)   # hand-written waits are inside
                waits = re.findall(r"s_waitcnt vmcnt\((\d+)\)", own)
                if waits:
                    found.append((parts[i][-70:], block.split(":")[0].strip(), waits))
    return kernels, found


def main() -> int:
    bad = 0
    with tempfile.TemporaryDirectory() as tmp:
        done = {}
        for src, kernel in FILES:
            if src not in done:
                done[src] = os.path.join(tmp, src + ".s")
                assembly(src, done[src])
            kernels, found = scan(open(done[src]).read(), kernel)
            print(f"{src}: {kernels} instantiations of {kernel}, {len(found)} main-loop blocks with a compiler wait")
            for name, label, waits in found:
                print(f"    ...{name} {label}: vmcnt {', '.join(waits)}")
            bad += len(found)
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
