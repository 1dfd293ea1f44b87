#!/usr/bin/env python3
"""Checks the compiled k loop of the one-wavefront-per-SIMD GEMM kernel (qgemm_bw.hpp).

Its MFMAs are inline assembly, so the compiler does not know that they complete late: any
instruction it places between them that reads or moves an accumulator (a register copy, a
spill to scratch) would read a register an MFMA is still writing.  The source is written so
that none is needed; this script verifies it on the generated ISA.

    hipcc --offload-arch=gfx950 ... --cuda-device-only -S qgemm_bw.hip -o bw.s
    python3 check_mfma_loop.py bw.s        # exit status 1 and a report if a loop is not clean
"""
import re
import sys


def check(asm_text: str) -> list[str]:
    """Returns one line per MFMA loop found: 'kernel: N mfma, clean' or the offending instructions."""
    report = []
    for m in re.finditer(r"^(_ZN[^\n:]*qgemm_bw_kernel[^\n:]*):[^\n]*\n(.*?)s_endpgm", asm_text, flags=re.S | re.M):
        name, body = m.group(1), m.group(2).splitlines()
        for i, line in enumerate(body):
            head = re.match(r"^(\.LBB\d+_\d+):.*Loop Header", line)
            if not head:
                continue
            for k in range(i + 1, len(body)):
                if re.search(r"s_cbranch_\w+ " + re.escape(head.group(1)) + r"\b", body[k]):
                    seg = body[i:k + 1]
                    n_mfma = sum("v_mfma" in s for s in seg)
                    if n_mfma >= 40:
                        bad = [s.strip() for s in seg if re.search(r"scratch_|v_accvgpr|v_mov_b32", s)]
                        report.append(f"{name}: {n_mfma} mfma, " + ("clean" if not bad else "NOT CLEAN: " + "; ".join(bad[:6])))
                    break
    return report


if __name__ == "__main__":
    rep = check(open(sys.argv[1]).read())
    print("\n".join(rep) if rep else "no MFMA loop found")
    sys.exit(0 if rep and all(r.endswith("clean") for r in rep) else 1)
