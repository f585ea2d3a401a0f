"""Compiles the HIP sources under csrc/ into csrc/libmfq.so for gfx950.

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain
is installed.  The library is built in-tree so that it travels with the
source tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB_PATH = os.path.join(CSRC, "libmfq.so")
SOURCES = ("abi.hip", "quantize.hip", "qmv.hip", "qmv_dot.hip", "qmv_quad.hip", "qmv_odd.hip", "qmv_oct.hip", "qmv_oct4.hip", "qmm.hip", "qmm_epi.hip", "qmm_mid.hip", "qmm_mid_stream.hip", "qmm_n.hip", "qmm_frag.hip", "lora.hip", "norm.hip")

# -ffp-contract=off, correctly rounded division and preserved denormals make
# the quantize kernel's float32 arithmetic the same IEEE operations as the
# scalar CPU algorithm.  Packed-FP32 instruction selection is switched off.
HIPCC_FLAGS = (
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt", "-fno-gpu-flush-denormals-to-zero",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-pragmas",
)


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the mfq library cannot be built")
    return exe


def _compile(src: str) -> str:
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{res.stdout}\n{res.stderr}")
    return obj


# Kernels whose matrix instructions are inline assembly (result tied to the addend), which the compiler's
# hazard recognizer cannot see: {source: substring of the kernels' mangled names}.
ASM_MFMA_KERNELS = {"qmm_frag.hip": "frag_gemm_kernel"}


def _parse_blocks(body: str):
    """A kernel's listing as basic blocks: [(label, [instruction lines])], split at every label line."""
    import re

    blocks = [("", [])]
    for ln in body.split("\n"):
        s = ln.strip()
        m = re.match(r"^(\.L[A-Za-z0-9_$.]+):", s)
        if m:
            blocks.append((m.group(1), []))
            continue
        if not s or s.startswith((";", ".")):
            continue
        blocks[-1][1].append(s)
    return blocks


def _wait_states(ins: str) -> int:
    """What an instruction puts between its neighbours: one issue slot, or the count of an s_nop."""
    if ins.startswith("s_nop"):
        return int(ins.split()[1], 0) + 1
    return 1


def check_listing(text: str, kernel_substring: str, where: str = "listing") -> int:
    """Checks every kernel of the assembly listing `text` whose name contains
    `kernel_substring` for what neither the hardware nor the compiler's hazard
    recognizer (which does not see matrix instructions written as assembly)
    would catch.  (1) and (2) follow the control flow: from each instruction
    they walk every path through the kernel's basic blocks (fall-through and
    both ways of each branch, back edges included) until the distance is used
    up, counting an s_nop by its wait states.
    (1) a read of an accumulation register (v_accvgpr_read, the source of a
    v_accvgpr_mov) or a write of one from outside the matrix pipeline
    (v_accvgpr_write, the destination of a _mov) must lie at least 24 wait
    states behind the last matrix instruction that wrote that register: the
    kernels touch accumulators either behind wait states of their own, or (the
    first pass of a tile, which stores the previous one) some sixty matrix
    instructions after the register's last update;
    (2) a matrix instruction that adds to a register must lie at least 4 wait
    states behind a write of that register from outside the pipeline;
    (3) the body of the k loop may not wait for its loads with a count below 8
    (6 with three column tiles per wavefront instead of four): the weight
    fragments are requested a step and a half ahead with at least nine (six)
    younger requests behind them, and a smaller count means that the
    compiler's wait counting entered the loop believing loads outstanding that
    are not, and waits for the newest requests instead (seen once, 20 us per
    call);
    (4) a kernel may spill at most 48 registers (the kernels use all 512 and
    spill a dozen or two outside the k loop; the compiler's choices around the
    assembly have tipped over into hundreds, with accumulators moved between
    the register files, on small changes to the source).
    Returns the number of kernels checked; raises RuntimeError on a finding."""
    import re

    checked = 0
    for m in re.finditer(r"^(\S*%s\S*):" % re.escape(kernel_substring), text, re.M):
        name = m.group(1)
        body = text[m.end():text.index(".Lfunc_end", m.end())]
        blocks = _parse_blocks(body)
        index = {label: i for i, (label, _) in enumerate(blocks) if label}
        col_tiles = re.search(r"ELi(\d)ELb[01]EEEv", name)  # the template argument before the last: column tiles per wavefront
        least = 2 * int(col_tiles.group(1)) if col_tiles else 8

        def successors(b):
            ins = blocks[b][1]
            out = []
            for s in ins:
                t = re.match(r"s_c?branch\S*\s+(\S+)", s)
                if t and t.group(1) in index:
                    out.append(index[t.group(1)])
            last = ins[-1] if ins else ""
            if not (last.startswith("s_branch") or last.startswith("s_endpgm") or last.startswith("s_setpc")):
                if b + 1 < len(blocks):
                    out.append(b + 1)
            return out

        def walk(b, i, budget, visit, seen):
            """Calls visit(instruction) for everything within `budget` wait states behind instruction i of block b."""
            ins = blocks[b][1]
            while budget > 0:
                i += 1
                if i >= len(ins):
                    for nb in successors(b):
                        if seen.get(nb, 0) < budget:  # not yet entered with as much distance left
                            seen[nb] = budget
                            walk(nb, -1, budget, visit, seen)
                    return
                visit(ins[i])
                budget -= _wait_states(ins[i])

        n_matrix = 0
        for b, (label, ins) in enumerate(blocks):
            matrix = sum(s.startswith("v_mfma") for s in ins)
            n_matrix += matrix
            if matrix >= 128:  # the k loop's body (an item's first step and the low-rank update are blocks of fewer)
                last_m = max(i for i, s in enumerate(ins) if s.startswith("v_mfma"))
                short = [int(c) for s in ins[:last_m] for c in re.findall(r"s_waitcnt vmcnt\((\d+)\)", s) if int(c) < least]
                if short:
                    raise RuntimeError(f"{where}: {name} waits with vmcnt({min(short)}) inside its k loop")
            for i, s in enumerate(ins):
                op = s.split()[0]
                if op.startswith("v_mfma"):
                    lo, hi = [(int(a), int(c)) for a, c in re.findall(r"a\[(\d+):(\d+)\]", s)][0]

                    def touches(t, lo=lo, hi=hi):
                        if t.startswith("v_accvgpr"):
                            for reg in re.findall(r"\ba(\d+)\b", t):
                                if lo <= int(reg) <= hi:
                                    raise RuntimeError(f"{where}: {name} touches a{reg} within 24 wait states of a matrix "
                                                       f"instruction that writes it")

                    walk(b, i, 24, touches, {})
                elif op.startswith("v_accvgpr_write") or op.startswith("v_accvgpr_mov"):
                    reg = int(re.findall(r"\ba(\d+)\b", s)[0])

                    def adds(t, reg=reg):
                        if t.startswith("v_mfma"):
                            ranges = [(int(a), int(c)) for a, c in re.findall(r"a\[(\d+):(\d+)\]", t)]
                            if len(ranges) > 1 and ranges[-1][0] <= reg <= ranges[-1][1]:
                                raise RuntimeError(f"{where}: {name}: a matrix instruction adds to a[{ranges[-1][0]}:"
                                                   f"{ranges[-1][1]}] within 4 wait states of a write to it")

                    walk(b, i, 4, adds, {})
        if not n_matrix:
            raise RuntimeError(f"{where}: {name} holds no matrix instruction; the check does not see the kernel")
        spills = re.search(r"\.name:\s+%s\n(?:.*\n)*?\s*\.vgpr_spill_count:\s*(\d+)" % re.escape(name), text)
        if spills is None or int(spills.group(1)) > 48:
            raise RuntimeError(f"{where}: {name} spills {spills and spills.group(1)} registers (at most 48 expected)")
        checked += 1
    if not checked:
        raise RuntimeError(f"{where}: no kernel named *{kernel_substring}* found")
    return checked


def check_generated_code(src: str) -> int:
    """Compiles `src` to assembly (device side) and runs check_listing over the
    kernels named in ASM_MFMA_KERNELS.  Returns the number of kernels checked;
    raises on a finding."""
    import tempfile

    with tempfile.TemporaryDirectory() as tmp:
        asm = os.path.join(tmp, "out.s")
        cmd = [hipcc(), *HIPCC_FLAGS, "--cuda-device-only", "-S", "-c", os.path.join(CSRC, src), "-o", asm]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc -S failed on {src}:\n{res.stdout}\n{res.stderr}")
        text = open(asm).read()
    return check_listing(text, ASM_MFMA_KERNELS[src], src)


def build_library(verbose: bool = False) -> str:
    """Always recompiles every translation unit, checks the generated code of the
    kernels in ASM_MFMA_KERNELS and relinks libmfq.so."""
    with ThreadPoolExecutor(max_workers=len(SOURCES) + len(ASM_MFMA_KERNELS)) as pool:
        checks = [pool.submit(check_generated_code, src) for src in ASM_MFMA_KERNELS]
        objs = list(pool.map(_compile, SOURCES))
        for c in checks:
            c.result()
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


def sanitize_abi(verbose: bool = False) -> str:
    """Host-sanitizer run of the C ABI's argument validation: abi.hip compiled
    with AddressSanitizer and UndefinedBehaviorSanitizer on its host side (the
    device side is untouched), linked with the ordinary kernel objects and the
    driver tests/abi_sanitize_check.cpp, and run.  Every call in the driver is
    refused before a launch, so no GPU is needed.  Needs the objects of
    build_library().  Returns the driver's output; raises if it reports a
    finding."""
    san = os.path.join(CSRC, "_san")
    os.makedirs(san, exist_ok=True)
    host_san = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
                "-Xarch_host", "-fno-sanitize-recover=all", "-Xarch_host", "-fno-omit-frame-pointer", "-g"]
    abi_o = os.path.join(san, "abi.o")
    drv_o = os.path.join(san, "abi_sanitize_check.o")
    exe = os.path.join(san, "abi_sanitize_check")
    others = [os.path.join(CSRC, os.path.splitext(s)[0] + ".o") for s in SOURCES if s != "abi.hip"]
    missing = [o for o in others if not os.path.exists(o)]
    if missing:
        raise RuntimeError(f"run build_library() first: {missing[0]} is missing")
    steps = [
        [hipcc(), *HIPCC_FLAGS, *host_san, "-c", os.path.join(CSRC, "abi.hip"), "-o", abi_o],
        [hipcc(), "-O1", "-g", "-std=c++17", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-c",
         os.path.join(os.path.dirname(os.path.dirname(CSRC)), "tests", "abi_sanitize_check.cpp"), "-o", drv_o],
        [hipcc(), "--offload-arch=gfx950", "-fsanitize=address,undefined", "-o", exe, drv_o, abi_o, *others],
    ]
    for cmd in steps:
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"{' '.join(cmd[:3])} ... failed:\n{res.stdout}\n{res.stderr}")
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:verify_asan_link_order=0", UBSAN_OPTIONS="print_stacktrace=1")
    res = subprocess.run([exe], capture_output=True, text=True, env=env)
    if res.returncode != 0:
        raise RuntimeError(f"abi_sanitize_check reported a finding (exit {res.returncode}):\n{res.stdout}\n{res.stderr}")
    if verbose:
        print(res.stdout.strip())
    return res.stdout


OPS_PATH = os.path.join(CSRC, "libmfq_torch.so")


def build_torch_ops(verbose: bool = False) -> str:
    """Compiles csrc/torch_ops.cpp (the torch.ops.mfq registrations, host C++
    only) against this interpreter's torch and links it to libmfq.so."""
    from torch.utils import cpp_extension

    torch_lib = cpp_extension.library_paths()[0]
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    tmp = OPS_PATH + ".tmp"
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=1", *[f"-I{p}" for p in cpp_extension.include_paths()], f"-I{rocm}/include",
           os.path.join(CSRC, "torch_ops.cpp"), "-o", tmp, f"-L{CSRC}", "-lmfq", f"-L{torch_lib}", "-ltorch",
           "-ltorch_cpu", "-lc10", "-ltorch_hip", "-lc10_hip", "-Wl,-rpath,$ORIGIN"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"g++ failed on torch_ops.cpp:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, OPS_PATH)
    if verbose:
        print(f"built {OPS_PATH}")
    return OPS_PATH


if __name__ == "__main__":
    import sys

    if "--sanitize-abi" in sys.argv:
        sanitize_abi(verbose=True)
    else:
        build_library(verbose=True)
        build_torch_ops(verbose=True)
