"""Build-time check of the compiled kernels for one matrix-instruction pairing that gfx950 gets wrong.

``v_mfma_f32_16x16x32_f16 D, ...`` followed by ``v_mfma_f32_16x16x16_f16 D, A, B, D`` (another opcode accumulating
on the first one's result) read a stale ``D`` in the first quarter of the wave when three or four other instructions
stood between the two, and the right one from five on (measured on MI355X, hipcc of ROCm 7.2: the compiler adds no
wait states for this pairing, and which distance a build gets depends on instruction scheduling).  The kernels keep
such pairs apart with ``mfma_shape_fence`` (csrc/chunk_common.h).  This module reads the assembly of a kernel and
reports every accumulator that passes from one MFMA opcode to another one with fewer than ``MIN_WAIT_STATES``
between them, so that a build which lost the fence, or gained a new pairing, fails instead of computing wrong values.
Pairs of the same opcode are left to the compiler: they are its ordinary case.
"""
import re

MIN_WAIT_STATES = 8


def _tuple(tok):
    m = re.match(r"v\[(\d+):(\d+)\]$", tok)
    if m:
        return int(m.group(1)), int(m.group(2))
    m = re.match(r"v(\d+)$", tok)
    return (int(m.group(1)),) * 2 if m else None


def scan(asm_text):
    """Returns [(wait_states, first_opcode, second_opcode, line)] for every MFMA whose accumulator input is the result
    of an MFMA with another opcode.  Wait states are counted as instructions in between, ``s_nop N`` as N + 1; the
    count restarts at every label (a branch target may be reached along a shorter path)."""
    last, wait, found = {}, 0, []
    for raw in asm_text.splitlines():
        line = raw.split(";")[0].strip()
        if not line or line.startswith("//") or (line.startswith(".") and not line.endswith(":")):
            continue
        if line.endswith(":"):
            for k in last:
                last[k] = (last[k][0], None)                 # distance unknown from here on
            continue
        op = line.split()[0]
        wait += int(line.split()[1]) + 1 if op == "s_nop" else 1
        operands = [o.strip() for o in line.split(None, 1)[1].split(",")] if " " in line or "\t" in line else []
        if op.startswith(("v_mfma", "v_smfmac")):
            dst = _tuple(operands[0])
            acc = _tuple(operands[3]) if len(operands) > 3 else None
            if acc is not None:
                for k, (prev_op, at) in last.items():
                    if prev_op != op and not (acc[1] < k[0] or acc[0] > k[1]):
                        found.append((None if at is None else wait - at - 1, prev_op, op, line))
            if dst is not None:
                for k in [k for k in last if not (dst[1] < k[0] or dst[0] > k[1])]:
                    del last[k]
                last[dst] = (op, wait)
        elif operands:
            dst = _tuple(operands[0])
            if dst is not None and not op.startswith(("ds_write", "global_store", "buffer_store", "v_cmp")):
                for k in [k for k in last if not (dst[1] < k[0] or dst[0] > k[1])]:
                    del last[k]
    return found


def violations(asm_text, min_wait=MIN_WAIT_STATES):
    return [f for f in scan(asm_text) if f[0] is None or f[0] < min_wait]


def check(asm_text, name, min_wait=MIN_WAIT_STATES):
    bad = violations(asm_text, min_wait)
    if bad:
        raise RuntimeError(
            "%s: an accumulator passes between MFMA opcodes with fewer than %d wait states:\n%s" %
            (name, min_wait, "\n".join("  %s wait states: %s -> %s" % (w, a, l) for w, a, _, l in bad)))
