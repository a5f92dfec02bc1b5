"""Builds muon_amd/libmuon_amd.so from muon_amd/csrc/*.hip with hipcc for gfx950.

    python -m muon_amd.build

After the library is built, the GEMM kernels are compiled once more to assembly and checked
(`check_fragment_waits`): their main loop requests its LDS fragments through inline assembly and
waits for them by hand, which is only correct while the compiler does not touch a requested
register before the wait that covers it.
"""
from __future__ import annotations

import os
import re
import shutil
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libmuon_amd.so")
SOURCES = ["capi.hip", "elementwise.hip", "aol.hip", "ns_gemm.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # hipcc -O3 must not form packed-fp32 instructions on this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


_VREG = re.compile(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b")


def _vregs(text: str) -> frozenset:
    out = set()
    for m in _VREG.finditer(text):
        if m.group(1):
            out |= set(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            out.add(int(m.group(3)))
    return frozenset(out)


def check_fragment_waits(asm_text: str) -> int:
    """Walks the control-flow graph of every ns_gemm_kernel in a hipcc -S listing.  A register that an
    inline-assembly LDS read (ds_read_b128, ds_read_b64_tr_b16) has requested is pending until a `s_waitcnt lgkmcnt(n)` leaves at
    most n younger requests outstanding (LDS reads return in order).  Raises if any instruction --
    a copy the register allocator put at a loop edge, an address computation, an MFMA -- names a
    pending register: it would see the register before its data.  Returns the number of such reads
    it followed."""
    lines = asm_text.split("\n")
    starts = [i for i, l in enumerate(lines) if re.match(r"^_ZN8muon_amd14ns_gemm_kernel\S*:", l)]
    if not starts:
        raise RuntimeError("check_fragment_waits: no ns_gemm_kernel in the listing")
    nreads = 0
    for k0 in starts:
        instrs, labels, inasm = [], {}, False
        for i in range(k0 + 1, len(lines)):
            t = lines[i].strip()
            if t.startswith(".Lfunc_end"):
                break
            if ";;#ASMSTART" in t:
                inasm = True
            elif ";;#ASMEND" in t:
                inasm = False
            elif re.match(r"^\.LBB\d+_\d+:", t):
                labels[t.split(":")[0]] = len(instrs)
            elif t and not t.startswith(";") and not t.startswith("."):
                instrs.append((t, inasm, i + 1))
        seen, stack = set(), [(0, ())]
        while stack:
            pc, pend = stack.pop()
            while pc < len(instrs) and (pc, pend) not in seen:
                seen.add((pc, pend))
                t, from_asm, line_no = instrs[pc]
                op = t.split()[0]
                if op == "s_waitcnt":
                    m = re.search(r"lgkmcnt\((\d+)\)", t)
                    if m:
                        n = int(m.group(1))
                        pend = pend[len(pend) - n:] if n else ()
                elif op in ("ds_read_b128", "ds_read_b64_tr_b16") and from_asm:
                    dst, addr = t.split(None, 1)[1].split(",")[:2]
                    if any(p & _vregs(addr) for p in pend):
                        raise RuntimeError(f"ns_gemm.hip: line {line_no} of the listing reads LDS through a pending register: {t}")
                    pend = pend + (_vregs(dst),)
                    nreads += 1
                elif op == "s_endpgm":
                    break
                elif op == "s_branch":
                    pc = labels[t.split()[1]]
                    continue
                else:
                    if op.startswith("s_cbranch"):
                        stack.append((labels[t.split()[1]], pend))
                    elif pend and any(p & _vregs(t) for p in pend):
                        raise RuntimeError(
                            f"ns_gemm.hip: line {line_no} of the listing touches a fragment register whose LDS read "
                            f"is still in flight: {t}")
                pc += 1
    if nreads == 0:
        raise RuntimeError("check_fragment_waits: the listing holds no inline-assembly fragment reads")
    return nreads


def build(verbose: bool = True, check: bool = True) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    tmp = OUT + ".tmp"
    cmd = [hipcc, *FLAGS, *[os.path.join(CSRC, s) for s in SOURCES], "-o", tmp]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("hipcc failed building libmuon_amd.so")
    if check:
        with tempfile.TemporaryDirectory() as d:
            listing = os.path.join(d, "ns_gemm.s")
            flags = [f for f in FLAGS if f not in ("-shared", "-fPIC")]
            cmd = [hipcc, *flags, "-S", "--cuda-device-only", os.path.join(CSRC, "ns_gemm.hip"), "-o", listing]
            proc = subprocess.run(cmd, capture_output=True, text=True)
            if proc.returncode != 0:
                sys.stderr.write(proc.stdout + proc.stderr)
                raise RuntimeError("hipcc failed writing the assembly listing of ns_gemm.hip")
            n = check_fragment_waits(open(listing).read())
            if verbose:
                print(f"ns_gemm.hip: {n} hand-waited fragment reads followed through the listing, none touched early", flush=True)
    os.replace(tmp, OUT)
    return OUT


if __name__ == "__main__":
    print(build())
