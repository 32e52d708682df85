"""What the compiler made of a kernel source's software pipelines: `python -m batchgen_amd.isa_audit gemm_fp8_skinny.hip`.

Compiles one file of csrc/ to gfx950 assembly (device side only) and prints, per kernel, the flat memory instructions
(there should be none: see build.py) and, for every innermost loop that holds workgroup barriers and matrix
instructions -- the prefetch rings -- the `s_waitcnt vmcnt(N)` values in program order.  A ring that keeps D stages in
flight shows counts of about D stages' worth of loads; a `0` inside such a loop is a full drain once per revolution
(hand-placed tail waits and item-boundary paths excepted) and is worth a look at the source: it is how the MXFP4
kernel's flat stores were found.  Reads this library's own kernels only.
"""
from __future__ import annotations

import os
import re
import subprocess
import sys
import tempfile

KERNEL = re.compile(r"^(_Z\w+): *;[^\n]*\n(.*?)^\s*s_endpgm", re.S | re.M)
LABEL = re.compile(r"^(\.LBB\d+_\d+):")
BRANCH = re.compile(r"s_c?branch\w* (\.LBB\d+_\d+)")
FLAT = re.compile(r"^\s*(flat_(?:load|store|atomic)\w*)", re.M)


def loops(body: list[str]) -> list[tuple[int, int]]:
    """(first, last) line of every backward branch's span."""
    at = {m.group(1): i for i, line in enumerate(body) if (m := LABEL.match(line))}
    out = []
    for i, line in enumerate(body):
        m = BRANCH.search(line)
        if m and m.group(1) in at and at[m.group(1)] < i:
            out.append((at[m.group(1)], i))
    return out


def audit(asm: str, min_barriers: int = 2, min_mfma: int = 8) -> list[dict]:
    """One record per kernel: name, flat instructions, and the wait counts of its innermost pipelined loops."""
    records = []
    for m in KERNEL.finditer(asm):
        body = [line.split(";")[0].rstrip() for line in m.group(2).splitlines()]
        spans = loops(body)

        def weight(a, b):
            seg = body[a:b + 1]
            return sum("s_barrier" in x for x in seg), sum("v_mfma" in x for x in seg)

        rings = []
        for a, b in spans:
            nb, nm = weight(a, b)
            if nb < min_barriers or nm < min_mfma:
                continue
            if any((a2, b2) != (a, b) and a2 >= a and b2 <= b and weight(a2, b2)[0] >= min_barriers for a2, b2 in spans):
                continue                                      # an outer loop: its rings are reported on their own
            waits = [int(w) for x in body[a:b + 1] for w in re.findall(r"vmcnt\((\d+)\)", x)]
            rings.append(dict(lines=(a, b), barriers=nb, mfma=nm, waits=waits))
        records.append(dict(kernel=m.group(1), flat=sorted(set(FLAT.findall(m.group(2)))), rings=rings))
    return records


def compile_to_asm(src: str) -> str:
    from batchgen_amd import build as b
    path = src if os.path.exists(src) else os.path.join(b.CSRC, src)
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "k.s")
        r = subprocess.run([b.hipcc()] + b.FLAGS + ["--cuda-device-only", "-S", "-c", path, "-o", out],
                           capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(r.stderr[-4000:])
        with open(out) as f:
            return f.read()


def main(argv: list[str]) -> int:
    if len(argv) != 2:
        print(__doc__)
        return 2
    for rec in audit(compile_to_asm(argv[1])):
        name = subprocess.run(["c++filt", rec["kernel"]], capture_output=True, text=True).stdout.strip() or rec["kernel"]
        name = re.sub(r"\(anonymous namespace\)::", "", name).split("(")[0]
        print(f"{name}: flat {rec['flat'] or 'none'}")
        seen = set()
        for ring in rec["rings"]:
            key = (ring["barriers"], ring["mfma"], tuple(ring["waits"]))
            if key in seen:
                continue
            seen.add(key)
            drained = " <- full wait inside the ring" if 0 in ring["waits"][1:] else ""
            print(f"    ring: {ring['barriers']} barriers, {ring['mfma']} MFMAs, vmcnt {ring['waits']}{drained}")
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
