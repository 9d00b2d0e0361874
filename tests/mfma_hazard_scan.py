"""Static check of the compiler's gfx950 assembly for one silent failure: a matrix-core (MFMA) result
read before it has been written.

An MFMA writes its destination registers ``passes`` issue slots after it starts (4 for the 16x16x32 f16
shape, 8 for 32x32x16), and the hardware does not stall an ordinary instruction that reads them earlier:
``passes + 2`` wait states have to lie between the two.  The compiler inserts ``s_nop`` for that inside a
basic block, but has been seen to emit a ``v_accvgpr_read`` two wait states after the MFMA when a taken
branch lay between them, which returned a stale score in paged attention.  ``scan`` walks every path
backwards from each reader (branches included) and reports readers that come too early.
"""
from __future__ import annotations

import collections
import re

_REG = re.compile(r"^([va])(?:(\d+)|\[(\d+):(\d+)\])$")
_STORES = ("global_store", "ds_write", "buffer_store", "scratch_store", "flat_store", "ds_bpermute", "ds_permute")
_LOOKBACK = 12  # wait states; more than the longest requirement (8 + 2)


def _regs(token: str) -> set:
    m = _REG.match(token)
    if not m:
        return set()
    kind = m.group(1)
    if m.group(2) is not None:
        return {(kind, int(m.group(2)))}
    return {(kind, i) for i in range(int(m.group(3)), int(m.group(4)) + 1)}


def _passes(opcode: str) -> int:
    return 8 if "32x32" in opcode else 4


def _functions(text: str):
    current, body = None, []
    for line in text.split("\n"):
        m = re.match(r"^(_Z\w+):", line)
        if m:
            current, body = m.group(1), []
            continue
        if line.startswith(".Lfunc_end"):
            if current:
                yield current, body
            current = None
            continue
        if current is not None:
            code = line.split(";")[0].rstrip()
            if code.strip():
                body.append(code)


def scan(asm_text: str) -> list:
    """Returns ``[(function, reader, wait_states, needed, mfma)]`` for every early read found."""
    found = []
    for name, body in _functions(asm_text):
        ins, labels = [], {}
        for code in body:
            m = re.match(r"^(\.LBB\w+):", code)
            if m:
                labels[m.group(1)] = len(ins)
            elif code.startswith("\t") and not code.strip().startswith("."):
                ins.append(code.strip().replace(",", " ").split())
        preds = collections.defaultdict(list)
        for i, t in enumerate(ins):
            if t[0] not in ("s_branch", "s_endpgm", "s_setpc_b64") and i + 1 < len(ins):
                preds[i + 1].append(i)
            if (t[0].startswith("s_cbranch") or t[0] == "s_branch") and t[-1] in labels:
                preds[labels[t[-1]]].append(i)
        if not any("mfma" in t[0] for t in ins):
            continue
        for i, t in enumerate(ins):
            op = t[0]
            if "mfma" in op or op.startswith("s_") or op.startswith("v_accvgpr_write"):
                continue
            operands = t[1:] if op.startswith(_STORES) else t[2:]
            sources = set()
            for tok in operands:
                sources |= _regs(tok)
            if not sources:
                continue
            seen, stack, worst = {}, [(p, 0) for p in preds[i]], None
            while stack:
                j, ws = stack.pop()
                if ws >= _LOOKBACK or seen.get(j, _LOOKBACK) <= ws:
                    continue
                seen[j] = ws
                tj = ins[j]
                if "mfma" in tj[0]:
                    need = _passes(tj[0]) + 2
                    if _regs(tj[1]) & sources:
                        if ws < need and (worst is None or ws < worst[0]):
                            worst = (ws, need, " ".join(tj))
                        continue
                    step = _passes(tj[0])
                elif tj[0] == "s_nop":
                    step = int(tj[1]) + 1
                else:
                    step = 1
                    written = _regs(tj[1]) if len(tj) > 1 and not tj[0].startswith(_STORES) else set()
                    if written and sources <= written:
                        continue  # every source was rewritten on this path after any MFMA
                stack.extend((p, ws + step) for p in preds[j])
            if worst:
                found.append((name, " ".join(t), worst[0], worst[1], worst[2]))
    return found
