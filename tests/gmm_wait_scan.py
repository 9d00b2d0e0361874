"""Static check of the compiler's gfx950 assembly of the persistent grouped-matmul kernel for what its
hand-counted synchronisation relies on and the compiler does not know about.

The kernel copies its operand tiles HBM/L2 -> LDS with ``global_load_lds_dwordx4`` written as inline asm, so
the compiler's own wait-count pass does not see the copies; the kernel waits for them itself with literal
``s_waitcnt`` immediates in front of bare ``s_barrier`` instructions:

* barrier B of a k tile follows the tile's activation copies (``kACopies`` per wave) and is preceded by a wait
  on LDS reads only ("preceded": in the same basic block, with nothing that touches memory or LDS in between);
* barrier A follows the weight copies (``kBCopies`` per wave) issued after barrier B and is preceded by
  ``s_waitcnt vmcnt(kBCopies) lgkmcnt(0)``: everything but the weight copies just issued has landed.  Vector
  memory operations complete in order, so other memory operations in between can only make that wait stricter;
  a copy that moved across a barrier, or a larger count, would let a wave read a tile that is not there yet or
  overwrite a stage that is still being read.
* every copy is the triple ``s_mov_b32 m0, <sgpr>`` / ``s_nop 0`` / ``global_load_lds_dwordx4`` (M0 carries the
  LDS address); nothing else in the kernel may write or read M0, which the compiler treats as reserved but does
  not protect across the asm.
* no register is spilled: reloading a spilled register needs ``s_waitcnt vmcnt(0)``, which would also wait for
  the next item's copies.

``scan`` returns a list of findings (empty = all of the above holds) and the number of barriers it checked.
"""
from __future__ import annotations

import collections
import re

COPY = "global_load_lds_dwordx4"
_MEMORY = ("global_", "ds_", "buffer_", "scratch_", "flat_", "s_load", "s_buffer_load", "s_store", "s_scratch")
# <MB, NB, WN, SWIGLU, GATHER, PROBE>; the measurement builds (PROBE != 0) leave copies out on purpose and are not checked
_KERNEL = re.compile(r"^_ZN4aops32grouped_matmul_persistent_kernelILi(\d+)ELi(\d+)ELi(\d+)ELb([01])ELb([01])ELi0EE")


def kernels(asm_text: str):
    """(name, body lines) of every persistent-kernel instantiation in the assembly."""
    current, body = None, []
    for line in asm_text.split("\n"):
        m = re.match(r"^(_Z\w+):", line)
        if m:
            current, body = m.group(1), []
            continue
        if line.startswith(".Lfunc_end"):
            if current and _KERNEL.match(current):
                yield current, body
            current = None
            continue
        if current is not None:
            code = line.split(";")[0].rstrip()
            if code.strip():
                body.append(code)


def copies_per_wave(name: str):
    """(kACopies, kBCopies) of an instantiation: tile rows / 8 rows per copy / waves."""
    mb, nb, wn = (int(g) for g in _KERNEL.match(name).groups()[:3])
    waves = 2 * wn
    return 64 * mb // 8 // waves, 32 * nb * wn // 8 // waves


def _wait_fields(tokens):
    text = " ".join(tokens[1:])
    out = {}
    for key in ("vmcnt", "lgkmcnt", "expcnt"):
        m = re.search(key + r"\((\d+)\)", text)
        if m:
            out[key] = int(m.group(1))
    if not out and len(tokens) > 1:  # a raw immediate: vmcnt = bits 3:0 and 15:14, lgkmcnt = bits 11:8
        imm = int(tokens[1], 0)
        out = {"vmcnt": (imm & 0xF) | ((imm >> 14) & 0x3) << 4, "lgkmcnt": (imm >> 8) & 0xF}
    return out


def scan_kernel(name: str, body) -> tuple:
    findings = []
    k_a, k_b = copies_per_wave(name)
    ins, labels = [], {}
    for code in body:
        m = re.match(r"^(\.LBB\w+):", code)
        if m:
            labels[m.group(1)] = len(ins)
        elif code.startswith("\t") and not code.strip().startswith("."):
            ins.append(code.strip().replace(",", " ").split())
    label_at = set(labels.values())
    preds = collections.defaultdict(list)
    for i, t in enumerate(ins):
        if t[0] not in ("s_branch", "s_endpgm", "s_setpc_b64") and i + 1 < len(ins):
            preds[i + 1].append(i)
        if (t[0].startswith("s_cbranch") or t[0] == "s_branch") and t[-1] in labels:
            preds[labels[t[-1]]].append(i)

    # M0: only the copy triple touches it
    for i, t in enumerate(ins):
        if "m0" not in t[1:]:
            continue
        ok = (t[0] == "s_mov_b32" and t[1] == "m0" and i + 2 < len(ins) and ins[i + 1][:2] == ["s_nop", "0"]
              and ins[i + 2][0] == COPY)
        if not ok:
            findings.append(f"{name}: M0 used outside a copy: {' '.join(t)}")
    for i, t in enumerate(ins):
        if t[0] == COPY and not (i >= 2 and ins[i - 2][:2] == ["s_mov_b32", "m0"] and ins[i - 1][:2] == ["s_nop", "0"]):
            findings.append(f"{name}: copy without its own M0 set-up at instruction {i}")
    # no spills
    for t in ins:
        if t[0].startswith("scratch_") or t[0].startswith("buffer_"):
            findings.append(f"{name}: scratch or buffer access: {' '.join(t)}")
            break

    # barriers: the wait in front, and the copies since the barrier before on every path
    barriers = 0
    for i, t in enumerate(ins):
        if t[0] != "s_barrier":
            continue
        barriers += 1
        # the wait belongs to the barrier: same basic block, and nothing that touches memory or LDS in between
        # (register moves the compiler places there are harmless)
        w = i - 1
        while w >= 0 and ins[w][0] != "s_waitcnt" and not ins[w][0].startswith(_MEMORY) and \
                not ins[w][0].startswith(("s_cbranch", "s_branch", "s_barrier")) and (w + 1) not in label_at and i - w < 24:
            w -= 1
        if w < 0 or ins[w][0] != "s_waitcnt" or any(j in label_at for j in range(w + 1, i + 1)):
            findings.append(f"{name}: s_barrier at instruction {i} without an s_waitcnt in front")
            continue
        wait = _wait_fields(ins[w])
        counts, at_entry = set(), set()
        seen, stack = set(), [(p, 0) for p in preds[i]]
        while stack:
            j, c = stack.pop()
            if (j, c) in seen or c > 64:
                continue
            seen.add((j, c))
            op = ins[j][0]
            if op == "s_barrier":
                counts.add(c)
                continue
            if op == COPY:
                c += 1
            if not preds[j]:
                at_entry.add(c)
                continue
            stack.extend((p, c) for p in preds[j])
        if "vmcnt" in wait:  # barrier A: the weight copies just issued may still be in flight, nothing else
            if wait["vmcnt"] != k_b or wait.get("lgkmcnt") != 0:
                findings.append(f"{name}: barrier at {i}: expected s_waitcnt vmcnt({k_b}) lgkmcnt(0), found {wait}")
            if counts - {k_b}:
                findings.append(f"{name}: barrier A at {i}: {sorted(counts)} copies since the barrier before, expected {k_b}")
            if at_entry - {2 * k_b + k_a}:  # kernel start: weights of tiles 0 and 1, activations of tile 0
                findings.append(f"{name}: first barrier at {i}: {sorted(at_entry)} copies since kernel start, "
                                f"expected {2 * k_b + k_a}")
        else:               # barrier B: waits for LDS reads only, follows the activation copies
            if "lgkmcnt" not in wait:
                findings.append(f"{name}: barrier at {i}: wait without lgkmcnt: {wait}")
            if counts - {k_a} or at_entry:
                findings.append(f"{name}: barrier B at {i}: {sorted(counts | at_entry)} copies since the barrier before, "
                                f"expected {k_a}")
    return findings, barriers


def scan(asm_text: str) -> tuple:
    findings, barriers, names = [], 0, []
    for name, body in kernels(asm_text):
        f, b = scan_kernel(name, body)
        findings += f
        barriers += b
        names.append(name)
    return findings, barriers, names


def private_segment_sizes(asm_text: str) -> dict:
    """kernel name -> bytes of scratch per lane, from the .amdhsa_kernel blocks."""
    out = {}
    for block in asm_text.split(".amdhsa_kernel ")[1:]:
        name = block.split("\n")[0].strip()
        m = re.search(r"\.amdhsa_private_segment_fixed_size (\d+)", block)
        if m and _KERNEL.match(name):
            out[name] = int(m.group(1))
    return out
