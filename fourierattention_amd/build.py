"""Build recipe for the HIP shared library (gfx950 only).

``python -m fourierattention_amd.build`` compiles every source under ``csrc/`` with
hipcc and links ``fourierattention_amd/libfourier_attn_hip.so`` in-tree.
"""
from __future__ import annotations

import glob
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_NAME = "libfourier_attn_hip.so"
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed FP32 VALU ops are kept off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
]


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def audit_async_lds_reads(asm_text: str):
    """Find instructions that touch the destination of an inline-asm LDS read before it has been waited for.

    The matrix-core kernels issue ``ds_read`` from inline asm and tie the ``s_waitcnt`` to the result later, so
    that the compiler does not wait for the asynchronous page loads at every read.  Until that wait the
    registers do not hold the data, but the compiler believes they do and is free to copy them (it does when a
    read under a condition is merged with the other path).  The copy reads stale registers and nothing fails at
    build time, so every build checks the generated assembly: between such a read and the ``lgkmcnt`` wait
    that covers it, no instruction outside an asm block may name its registers.  The scan follows the layout of the
    code, not its control flow: it runs straight through conditional branches and starts afresh behind an
    unconditional one.  Returns the violations."""
    def regs(text):
        out = set()
        for m in re.finditer(r"\bv\[(\d+):(\d+)\]", text):
            out.update(range(int(m.group(1)), int(m.group(2)) + 1))
        for m in re.finditer(r"\bv(\d+)\b", text):
            out.add(int(m.group(1)))
        return out

    kernel, in_asm, pending, found = None, False, [], []   # pending: (registers, line) in issue order
    for no, line in enumerate(asm_text.split("\n"), 1):
        mk = re.match(r"^(_Z\S+):", line)
        if mk:
            kernel, pending = mk.group(1), []
        s = line.strip()
        if "ASMSTART" in s:
            in_asm = True
            continue
        if "ASMEND" in s:
            in_asm = False
            continue
        if not s or s[0] in ";.":
            continue
        m = re.match(r"(\S+)\s*(.*)", s.split(";")[0])
        if not m:
            continue
        op, args = m.group(1), m.group(2)
        if op in ("s_branch", "s_endpgm", "s_setpc_b64"):
            # what follows is not reached by falling through: it is another block laid out here (a loop's exit
            # after its body), entered from places of its own with their own outstanding reads
            pending = []
            continue
        if op == "s_waitcnt":
            mm = re.search(r"lgkmcnt\((\d+)\)", args)
            if mm:   # LDS operations complete in issue order: all but the last n are done
                n = int(mm.group(1))
                pending = pending[len(pending) - n:] if n else []
            continue
        if in_asm and op.startswith("ds_read"):
            pending.append((regs(args.split(",")[0]), no))
            continue
        if op.startswith("ds_") or op.startswith("s_load") or op.startswith("s_buffer_load"):
            pending.append((set(), no))   # shares the counter
        if in_asm:
            continue
        used = regs(args)
        for dst, at in pending:
            if dst & used:
                found.append(f"{kernel}: line {no} `{s[:80]}` touches v{sorted(dst & used)} of the read at line {at}")
                break
    return found


# kernels in which one workgroup hands data to another inside a launch: it stores, waits for the stores, then counts
# itself in with an atomic (decode_merge_rows_kernel; the instances of decode_mid_mfma_kernel that merge their own
# partials: the third from last of their template arguments, FUSE, is `true`)
HANDOVER_KERNELS = (re.compile(r"decode_merge_rows_kernel"), re.compile(r"decode_mid_mfma_kernel\S*Lb1ELb[01]ELb[01]EEEv"))
_STORE_OPS = ("global_store", "buffer_store", "flat_store")


def audit_handover_stores(asm_text: str, kernels=HANDOVER_KERNELS):
    """In the kernels that hand data from one workgroup to another, every counting atomic must find the workgroup's
    stores acknowledged: walking back from each ``global_atomic_add`` through the listing, an ``s_waitcnt`` with
    ``vmcnt(0)`` has to come before any vector-memory store does.  The source guarantees it (``s_waitcnt(0)``, a
    barrier, then the atomic), but nothing in the language ties the stores to that wait: a compiler that sank a store
    below it would produce a hand-over that works most of the time.  Returns ``(violations, atomics_seen)``; the scan
    follows the layout of the code backwards (labels and branches are passed over), which is conservative for the
    straight-line sequences it is meant for."""
    found, seen = [], 0
    lines = asm_text.split("\n")
    kernel, start = None, 0
    for no, line in enumerate(lines):
        mk = re.match(r"^(_Z\S+):", line)
        if mk:
            kernel, start = mk.group(1), no
            continue
        if kernel is None or not any(k.search(kernel) for k in kernels):
            continue
        s_ = line.strip().split(";")[0].strip()
        if not s_.startswith("global_atomic_add"):
            continue
        seen += 1
        ok = False
        for back in range(no - 1, start, -1):
            t = lines[back].strip().split(";")[0].strip()
            if not t or t.startswith("."):
                continue
            if t.startswith("s_waitcnt") and re.search(r"vmcnt\(0\)", t):
                ok = True
                break
            if t.startswith(_STORE_OPS):
                found.append(f"{kernel}: the atomic at line {no + 1} follows `{t[:70]}` (line {back + 1}) with no "
                             "s_waitcnt vmcnt(0) in between")
                ok = True   # reported
                break
        if not ok:
            found.append(f"{kernel}: no s_waitcnt vmcnt(0) in front of the atomic at line {no + 1}")
    return found, seen


# sources whose kernels issue LDS reads from inline asm (directly or through fa_decode_mfma.h): their assembly must
# show such reads, or the audit above has looked at nothing
def kernels_with_atomics_outside(asm_text: str, kernels=HANDOVER_KERNELS):
    """Kernels of a listing that issue a ``global_atomic_add`` but are not among the kernels ``audit_handover_stores``
    looks at: a hand-over the audit does not know of (a new kernel, or a kernel whose name no longer matches)."""
    out, kernel = [], None
    for line in asm_text.split("\n"):
        mk = re.match(r"^(_Z\S+):", line)
        if mk:
            kernel = mk.group(1)
            continue
        if kernel and line.strip().startswith("global_atomic_add") and not any(k.search(kernel) for k in kernels):
            if kernel not in out:
                out.append(kernel)
    return out


ASYNC_LDS_SOURCES = ("fa_decode_mid_bf16", "fa_decode_mid_f16", "fa_prefill", "fa_spectral_mfma")
HANDOVER_SOURCES = ("fa_decode", "fa_decode_mid_bf16", "fa_decode_mid_f16")


def count_async_lds_reads(asm_text: str) -> int:
    """Inline-asm ``ds_read`` instructions in a gfx950 assembly listing (what ``audit_async_lds_reads`` follows)."""
    n, in_asm = 0, False
    for line in asm_text.split("\n"):
        s = line.strip()
        if "ASMSTART" in s:
            in_asm = True
        elif "ASMEND" in s:
            in_asm = False
        elif in_asm and s.startswith("ds_read"):
            n += 1
    return n


def audit_listings(base: str, listings) -> list:
    """The audit of one source file, failing closed: ``listings`` are the texts of the gfx950 assembly files the
    compile left behind.  None at all, or none of the expected inline-asm reads in a source that uses them, is
    reported like a violation (the scan would otherwise pass by not seeing anything)."""
    if not listings:
        return [f"{base}: the compile left no gfx950 assembly listing to audit"]
    found, reads = [], 0
    for text in listings:
        found += audit_async_lds_reads(text)
        reads += count_async_lds_reads(text)
    if base in ASYNC_LDS_SOURCES and reads == 0:
        found.append(f"{base}: no inline-asm LDS read found in the assembly of a source that issues them "
                     "(markers or spellings the scan relies on have changed)")
    if base in HANDOVER_SOURCES:
        atomics = 0
        for text in listings:
            bad, n = audit_handover_stores(text)
            found += bad
            atomics += n
        if atomics == 0:
            found.append(f"{base}: no counting atomic found in the kernels that hand data between workgroups "
                         "(kernel names or spellings the scan relies on have changed)")
        for text in listings:
            for k in kernels_with_atomics_outside(text):
                found.append(f"{base}: {k} issues a counting atomic but is not among the kernels whose hand-over is audited")
    return found


def _compile(src: str, obj_dir: str, extra) -> str:
    base = os.path.basename(src)[:-4]
    obj = os.path.join(obj_dir, base + ".o")
    cmd = [HIPCC, *FLAGS, *extra, "-save-temps=obj", "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    listings = []
    for tmp in glob.glob(os.path.join(obj_dir, base + "-*")) + glob.glob(os.path.join(obj_dir, base + ".hip-*")):
        if tmp.endswith("gfx950.s"):
            with open(tmp) as f:
                listings.append(f.read())
        os.remove(tmp)   # intermediate files of the compile
    found = audit_listings(base, listings)
    if found:
        raise RuntimeError(f"{src}: the audit of the generated assembly failed:\n" + "\n".join(found))
    return obj


def build(verbose: bool = True, extra_flags=()) -> str:
    obj_dir = os.path.join(PKG_DIR, "build")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(lambda s: _compile(s, obj_dir, list(extra_flags)), srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources")
    return LIB_PATH


if __name__ == "__main__":
    build(extra_flags=sys.argv[1:])
