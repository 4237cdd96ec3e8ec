#!/usr/bin/env python3
"""Static check of the compiled kernels: wait states between a matrix instruction and the readers of its result.

On gfx950 nothing in the hardware holds back a vector, LDS or memory instruction that touches the result
registers of an MFMA which is still in the matrix pipe: the program has to let `passes + 4` issue slots go by
(12 for the 32x32x16 instructions used here).  The compiler inserts `s_nop`s for this, but it counts the slots
along one path only when the block that holds the MFMA reaches the reader by two paths of different length
(a conditional branch that skips a few scalar instructions), and it knows nothing about MFMAs written as inline
assembly.  Both have produced kernels that returned wrong values for the registers an MFMA writes last.

The script walks every path from every MFMA (fall-through and branch targets) through device assembly
(`hipcc -S --cuda-device-only`) until the required slots have gone by, counting one slot per instruction,
n + 1 for `s_nop n`, and the time a following MFMA waits for the matrix pipe, and reports every instruction on
the way that touches the result registers (for a following MFMA: that reads them as its A or B operand).

    python3 check_mfma_waits.py build/asm/*.s        (exit status 1 if anything is reported)
    make check-waits                                 (emits the assembly of every unit first)
"""
import re
import sys

_REG = re.compile(r"\b([va])(?:(\d+)|\[(\d+):(\d+)\])")
# passes (of four cycles) a matrix instruction keeps the pipe; only the shapes this library uses
_PASSES = {"32x32x16": 8, "16x16x32": 4}
_MEMORY = ("v_", "ds_", "global_", "buffer_", "flat_", "scratch_")


def _registers(operand):
    out = set()
    for m in _REG.finditer(operand):
        if m.group(2) is not None:
            out.add((m.group(1), int(m.group(2))))
        else:
            out.update((m.group(1), i) for i in range(int(m.group(3)), int(m.group(4)) + 1))
    return out


def _is_mfma(op):
    return op.startswith("v_mfma") or op.startswith("v_smfmac")


def _passes(op):
    for shape, n in _PASSES.items():
        if shape in op:
            return n
    raise ValueError(f"matrix instruction of unknown length: {op}")


def parse(text):
    """(instructions, labels): instructions as (text, opcode, operands, function); labels -> index."""
    instructions, labels, function = [], {}, None
    for line in text.split("\n"):
        s = line.split(";")[0].strip()
        if not s:
            continue
        m = re.match(r"^([.\w$]+):", s)
        if m:
            labels[m.group(1)] = len(instructions)
            if not m.group(1).startswith(".L"):
                function = m.group(1)
            continue
        if s.startswith("."):
            continue
        parts = s.split(None, 1)
        operands = [o.strip() for o in parts[1].split(",")] if len(parts) > 1 else []
        instructions.append((s, parts[0], operands, function))
    return instructions, labels


def report(found, key, entry):
    if key not in found or entry[3] < found[key][3]:
        found[key] = entry  # (the shortest of the paths that lead here)


def check(text):
    """List of (function, mfma text, reader text, slots waited) for every early access."""
    ins, labels = parse(text)
    n = len(ins)
    found = {}
    for i, (s, op, ops, fn) in enumerate(ins):
        if not _is_mfma(op):
            continue
        result = _registers(ops[0])
        need = _passes(op) + 4
        stack = [(i + 1, 0, _passes(op))]  # (index, slots gone by, slot at which the matrix pipe is free)
        best = {}
        while stack:
            j, w, free = stack.pop()
            while j < n and w < need:
                if best.get(j, need) <= w:
                    break
                best[j] = w
                s2, op2, ops2, _ = ins[j]
                if op2 == "s_endpgm":
                    break
                if _is_mfma(op2):
                    w = max(w, free)  # one instruction at a time in the matrix pipe
                    if w >= need:
                        break
                    free = w + _passes(op2)
                    if (_registers(ops2[1]) | _registers(ops2[2])) & result:
                        report(found, (i, j), (fn, s, s2, w))
                elif op2.startswith(_MEMORY):
                    touched = set()
                    for o in ops2:
                        touched |= _registers(o)
                    if touched & result:
                        report(found, (i, j), (fn, s, s2, w))
                w += int(ops2[0], 0) + 1 if op2 == "s_nop" else 1
                if op2 == "s_branch":
                    j = labels.get(ops2[0], n)
                    continue
                if op2.startswith("s_cbranch") and ops2[0] in labels:
                    stack.append((labels[ops2[0]], w, free))
                if op2 in ("s_setpc_b64", "s_swappc_b64"):
                    break
                j += 1
    return list(found.values())


def main(paths):
    total = 0
    for path in paths:
        with open(path) as f:
            found = check(f.read())
        print(f"{path}: {len(found)} early accesses")
        for fn, mfma, reader, waited in found[:20]:
            print(f"    {fn}: {mfma}  ->  {reader}  after {waited} slots")
        total += len(found)
    return 1 if total else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
