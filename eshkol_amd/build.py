"""Build libeshkol_gpu_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m eshkol_amd.build            # build into eshkol_amd/lib/
    python -m eshkol_amd.build --force    # rebuild even if up to date

Each source is compiled to an object under eshkol_amd/lib/obj/ and linked into
one shared library whose exported symbols are the C ABI declared in
include/eshkol/backend/gpu/gpu_memory.h and gpu_hip_tiers.h.
"""
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIBDIR = os.path.join(PKG, "lib")
OBJDIR = os.path.join(LIBDIR, "obj")
LIB = os.path.join(LIBDIR, "libeshkol_gpu_hip.so")

SOURCES = [
    "gpu_memory_hip.cpp",
    "host_copy.cpp",
    "dgemm_f64.hip",
    "dgemv_f64.hip",
    "dgemm_thin_f64.hip",
    "dgemm_small_f64.hip",
    "sgemm_f32.hip",
    "igemm_i8.hip",
    "igemm_thin_i8.hip",
    "hgemm_16.hip",
    "ozaki_crt.hip",
    "ozaki_int8.hip",
    "elementwise.hip",
    "ozaki_fast.hip",
]
# A device probe for the benchmark (register-only MFMA loops, a large copy): a
# library of its own, so that the product library carries no measurement code.
PROBE_LIB = os.path.join(LIBDIR, "libeshkol_gpu_probe.so")
PROBE_SOURCES = ["peak_probe.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# On gfx950 the fp64 MFMA runs at half rate when its accumulator lives in the
# AGPR half of the register file (measured: 36 vs 78 TFLOP/s on a register-only
# loop); the int8 and 16-bit MFMAs do not care. Keep fp64 accumulators in VGPRs.
EXTRA = {"dgemm_f64.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
         "dgemm_thin_f64.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
         "peak_probe.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}

# -ffp-contract=off: every fused multiply-add the arithmetic relies on is
# written as fma(); the compiler must not add or remove any.
# packed-fp32-ops is switched off for all device code in this library.
COMMON = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


# Kernels whose main loop issues its loads from inline assembly (gemm_pipe2.h): a
# register the compiler spills while such a load is still in flight would be saved
# before its data has arrived. They must therefore compile without any vector
# spill; the compiler's resource remarks are checked after every build.
NO_SPILL = {"igemm_i8.hip": ["igemm_i8_direct_kernel", "igemm_i8_direct_half_kernel"], "hgemm_16.hip": ["hgemm_direct_kernel"]}


def _check_no_spill(src, remarks):
    wanted = NO_SPILL.get(src, [])
    current, seen = None, set()
    for line in remarks.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split()[0]
            current = next((w for w in wanted if w in name), None)
            if current:
                seen.add(current)
        elif current and ("ScratchSize" in line or "VGPRs Spill" in line):
            value = int(line.split(":")[-1].split("[")[0].strip())
            if value != 0:
                raise RuntimeError("%s: kernel %s spills vector registers (%s); its asynchronous loads "
                                   "do not survive that" % (src, current, line.strip()))
    missing = [w for w in wanted if w not in seen]
    if missing:
        raise RuntimeError("%s: no resource remarks for %s; cannot prove it is free of spills" % (src, missing))


def sgpr_to_vmem_hazards(asm):
    """Places in gfx9 assembly text where a memory instruction reads a scalar
    register fewer than five wait states after a vector instruction wrote it
    (v_readlane of a spilled scalar, v_readfirstlane, a compare). The compiler
    keeps that distance between its own instructions; it does not look inside an
    asm statement, so a memory instruction issued from one can land right behind
    the reload of its address. Returns a list of (line number, text, wait states)."""
    def sregs(tok):
        m = re.fullmatch(r"s(\d+)", tok)
        if m:
            return {int(m.group(1))}
        m = re.fullmatch(r"s\[(\d+):(\d+)\]", tok)
        if m:
            return set(range(int(m.group(1)), int(m.group(2)) + 1))
        return set()
    pending, found = [], []
    for no, raw in enumerate(asm.split("\n"), 1):
        line = raw.split(";")[0].strip()
        if not line or line.endswith(":") or line.startswith("."):
            continue
        parts = line.replace(",", " ").split()
        op, ops = parts[0], parts[1:]
        if op.startswith(("buffer_", "global_", "flat_", "scratch_")):
            used = set()
            for t in ops:
                used |= sregs(t)
            for regs, ws, _ in pending:
                if regs & used and ws < 5:
                    found.append((no, line, ws))
        step = int(ops[0]) + 1 if op == "s_nop" and ops else 1
        pending = [(r, ws + step, l) for (r, ws, l) in pending if ws + step < 5]
        if op.startswith("v_") and ops and sregs(ops[0]):
            pending.append((sregs(ops[0]), 0, no))
    return found


def hidden_load_violations(asm, kernels, limit=400000):
    """Places in gfx9 assembly text where an instruction of one of the named kernels touches
    a vector register that a vector memory load may still be writing. The kernels of
    gemm_pipe2.h issue their loads from asm statements and wait for them with hand-counted
    `s_waitcnt vmcnt(N)`, so the compiler neither knows that a ring register's value arrives
    late nor checks the counts: a copy of such a register that the compiler places before the
    wait (v_mov, v_accvgpr_write, a spill), or a count that is too large, would use stale data
    with no error. The model is the hardware's: loads return in issue order, so after
    vmcnt(N) every load but the N youngest has landed (stores share the counter but only make
    a wait stricter); loads into LDS hold a place in that order and write no register. Every
    path of the control-flow graph is followed, a state being the ordered destinations of the
    loads in flight. Returns a list of (kernel, line number, text, registers). What this does
    not see is whether a load INTO LDS has landed before the barrier that publishes it: that
    rests on the counts and on the bit-exact tests."""
    def vregs(tok):
        m = re.fullmatch(r"v(\d+)", tok)
        if m:
            return frozenset({int(m.group(1))})
        m = re.fullmatch(r"v\[(\d+):(\d+)\]", tok)
        if m:
            return frozenset(range(int(m.group(1)), int(m.group(2)) + 1))
        return frozenset()

    bodies, cur = {}, None
    for no, raw in enumerate(asm.split("\n"), 1):
        text = raw.split(";")[0].strip()
        if text.endswith(":") and not text.startswith(".") and not raw.startswith(("\t", " ")):
            cur = text[:-1] if any(k in text for k in kernels) else None
            if cur:
                bodies[cur] = []
        elif cur is not None:
            if text.startswith((".end_amdhsa_kernel", ".Lfunc_end")):
                cur = None
            elif text:
                bodies[cur].append((no, text))

    found = []
    for kernel, body in bodies.items():
        blocks, label_at, block = [], {}, []
        for no, text in body:
            if text.endswith(":"):
                if block:
                    blocks.append(block)
                    block = []
                label_at[text[:-1]] = len(blocks)
            elif not text.startswith("."):
                block.append((no, text))
                op = text.split()[0]
                if op in ("s_branch", "s_endpgm") or op.startswith("s_cbranch"):
                    blocks.append(block)
                    block = []
        if block:
            blocks.append(block)
        seen, work, bad = set(), [(0, ())], {}
        while work:
            bi, state = work.pop()
            if (bi, state) in seen or bi >= len(blocks):
                continue
            seen.add((bi, state))
            if len(seen) > limit:
                raise RuntimeError("%s: too many pipeline states to follow" % kernel)
            fifo, succ = list(state), None
            for no, text in blocks[bi]:
                parts = text.replace(",", " ").split()
                op, ops = parts[0], parts[1:]
                if op == "s_waitcnt":
                    m = re.search(r"vmcnt\((\d+)\)", text)
                    if m and len(fifo) > int(m.group(1)):
                        fifo = fifo[len(fifo) - int(m.group(1)):]
                    continue
                used = frozenset().union(*[vregs(t) for t in ops]) if ops else frozenset()
                if used:
                    for regs in fifo:
                        if regs & used:
                            bad.setdefault(no, (text, sorted(regs & used)))
                            break
                if op.startswith(("buffer_load", "global_load", "flat_load", "scratch_load")):
                    fifo.append(frozenset() if "lds" in ops else vregs(ops[0]))
                    fifo = fifo[-63:]                     # the counter saturates there; older loads have landed
                if op == "s_endpgm":
                    succ = []
                elif op == "s_branch":
                    succ = [label_at[ops[0]]]
                elif op.startswith("s_cbranch"):
                    succ = [label_at[ops[0]], bi + 1]
            for t in ([bi + 1] if succ is None else succ):
                work.append((t, tuple(fifo)))
        found += [(kernel, no) + v for no, v in sorted(bad.items())]
    return found


def _check_hazards(src):
    """Compiles src to assembly with the flags of the build and scans it."""
    path = os.path.join(CSRC, src)
    cmd = [HIPCC] + COMMON + EXTRA.get(src, []) + ["-x", "hip", "-S", "--cuda-device-only", path, "-o", "-"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc -S failed for %s:\n%s" % (src, res.stderr))
    found = sgpr_to_vmem_hazards(res.stdout)
    if found:
        raise RuntimeError("%s: memory instructions read scalar registers too soon after a vector instruction "
                           "wrote them:\n%s" % (src, "\n".join("  line %d: %s (%d wait states)" % f for f in found[:10])))
    late = hidden_load_violations(res.stdout, NO_SPILL[src])
    if late:
        raise RuntimeError("%s: registers are used while a load issued from an asm statement may still be writing "
                           "them:\n%s" % (src, "\n".join("  %s line %d: %s %s" % f for f in late[:10])))


def _newer(target, deps):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(d) <= t for d in deps)


def _compile(src, force):
    path = os.path.join(CSRC, src)
    obj = os.path.join(OBJDIR, os.path.splitext(src)[0] + ".o")
    headers = [os.path.join(CSRC, h) for h in os.listdir(CSRC) if h.endswith(".h")]
    headers += [os.path.join(ROOT, "include", "eshkol", "backend", "gpu", h)
                for h in ("gpu_memory.h", "gpu_hip_tiers.h", "gpu_hip_testing.h")]
    if not force and _newer(obj, [path] + headers):
        return obj
    cmd = [HIPCC] + COMMON + EXTRA.get(src, []) + ["-x", "hip", "-c", path, "-o", obj]
    if src in NO_SPILL:
        cmd.insert(1, "-Rpass-analysis=kernel-resource-usage")
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, res.stdout, res.stderr))
    if src in NO_SPILL:
        try:
            _check_no_spill(src, res.stderr)
        except RuntimeError:
            os.remove(obj)
            raise
    return obj


def build(force=False, verbose=False):
    os.makedirs(OBJDIR, exist_ok=True)
    stale = [s for s in NO_SPILL if force or not _newer(LIB, [os.path.join(CSRC, f) for f in os.listdir(CSRC)])]
    with ThreadPoolExecutor(max_workers=8) as pool:
        checks = [pool.submit(_check_hazards, s) for s in stale]      # the kernels that issue loads from asm
        objs = list(pool.map(lambda s: _compile(s, force), SOURCES + PROBE_SOURCES))
        for c in checks:
            c.result()
    for lib, members in ((LIB, objs[:len(SOURCES)]), (PROBE_LIB, objs[len(SOURCES):])):
        if force or not _newer(lib, members):
            cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + members + ["-ldl", "-lpthread"]
            res = subprocess.run(cmd, capture_output=True, text=True)
            if res.returncode != 0:
                raise RuntimeError("link failed:\n%s\n%s" % (res.stdout, res.stderr))
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv, verbose=True)
