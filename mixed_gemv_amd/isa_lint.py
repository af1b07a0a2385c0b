"""Checks the compiled gfx950 code of this library for two hazards the compiler cannot see.

The VALU kernel issues its dot products as inline assembly (`v_dot2c_f32_f16_dpp` /
`v_dot2c_f32_bf16_dpp`): the compiler knows neither that they read their first source through
DPP nor that they are dot instructions, so it pads neither hazard of this target:

  * a VGPR written by a VALU instruction must not be read through DPP within 2 wait states;
  * the result of a dot instruction must not be read by any other kind of instruction -- nor
    as a multiplicand by another dot -- within 3 wait states, nor be overwritten by another
    kind of VALU instruction within 2.

The sources keep the hazards away by construction (activation registers come straight from
loads; an `s_nop` settles each accumulator chain), but a register copy placed by the register
allocator in the middle of a chain would break that silently.  This module reads the assembly
the build keeps (`hipcc -save-temps`) and reports every place where one of the rules is
violated or cannot be shown to hold, so the build can refuse a library that has one.

Wait states: every instruction issued in between counts one, `s_nop N` counts N + 1.
"""
import json
import os
import re
import sys

DOT_RE = re.compile(r"^v_dot\w*")
REG_RE = re.compile(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]")
LABEL_RE = re.compile(r"^([.\w$]+):")
VALU_NO_VGPR_DST = ("v_cmp", "v_readlane", "v_readfirstlane")
DPP_WAIT_STATES = 2
DOT_READ_WAIT_STATES = 3
DOT_OVERWRITE_WAIT_STATES = 2


def _regs(text):
    out = set()
    for m in REG_RE.finditer(text):
        if m.group(1) is not None:
            out.add(int(m.group(1)))
        else:
            out.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return out


class Inst:
    __slots__ = ("op", "operands", "line", "text")

    def __init__(self, op, operands, line, text):
        self.op, self.operands, self.line, self.text = op, operands, line, text

    @property
    def is_dot(self):
        return bool(DOT_RE.match(self.op))

    @property
    def is_dpp(self):
        return "_dpp" in self.op or any(t in self.text for t in ("row_newbcast", "quad_perm", "row_shr", "row_shl",
                                                                  "row_ror", "row_bcast", "row_mirror", "row_half_mirror",
                                                                  "wave_shr", "wave_shl", "wave_ror", "wave_rol"))

    @property
    def is_valu(self):
        return self.op.startswith("v_")

    @property
    def wait_states(self):
        if self.op == "s_nop":
            try:
                return int(self.operands[0], 0) + 1
            except (IndexError, ValueError):
                return 1
        return 1

    def vgpr_writes(self):
        """VGPRs a VALU instruction writes (loads write theirs asynchronously and are guarded by waitcnt)."""
        if not self.is_valu or self.op.startswith(VALU_NO_VGPR_DST) or not self.operands:
            return set()
        return _regs(self.operands[0])

    def vgpr_reads(self):
        if self.is_valu and not self.op.startswith(VALU_NO_VGPR_DST):
            srcs = self.operands[1:]
            if self.is_dot or self.op.startswith(("v_mac", "v_fmac", "v_pk_fmac")):   # tied accumulator
                srcs = self.operands
            return set().union(*[_regs(o) for o in srcs]) if srcs else set()
        if self.op.startswith(("buffer_load", "global_load", "flat_load", "scratch_load", "ds_read", "s_")):
            ops = self.operands[1:] if not self.op.startswith("s_") else self.operands
            return set().union(*[_regs(o) for o in ops]) if ops else set()
        return set().union(*[_regs(o) for o in self.operands]) if self.operands else set()


def parse_functions(path):
    """-> {function name: (blocks, order)}: blocks maps a label to its instructions, order lists the labels."""
    functions, name, blocks, order, cur = {}, None, None, None, None
    with open(path, errors="replace") as f:
        for ln, raw in enumerate(f, 1):
            line = raw.split(";", 1)[0].strip() if not raw.lstrip().startswith(";") else ""
            if not line:
                continue
            m = LABEL_RE.match(line)
            if m:
                label = m.group(1)
                if not label.startswith(".L"):
                    if name is not None:
                        functions[name] = (blocks, order)
                    name, blocks, order = label, {}, []
                if name is not None:
                    cur = label
                    blocks[cur] = []
                    order.append(cur)
                continue
            if line.startswith(".") or name is None or cur is None:
                if line.startswith(".end_amdhsa_kernel") or line.startswith(".section"):
                    pass
                continue
            parts = line.split(None, 1)
            op = parts[0]
            operands = [o.strip() for o in re.split(r",(?![^\[]*\])", parts[1])] if len(parts) > 1 else []
            # modifiers (row_newbcast:3 ...) ride on the last operand: keep only its first token there
            if operands:
                operands[-1] = operands[-1].split()[0] if operands[-1].split() else operands[-1]
            blocks[cur].append(Inst(op, operands, ln, line))
    if name is not None:
        functions[name] = (blocks, order)
    return functions


def _successors(blocks, order, label):
    insts = blocks[label]
    succ = []
    last = insts[-1] if insts else None
    falls = True
    if last is not None:
        if last.op == "s_branch":
            falls = False
            succ.append(last.operands[0])
        elif last.op.startswith("s_cbranch"):
            succ.append(last.operands[0])
        elif last.op in ("s_endpgm", "s_setpc_b64"):
            falls = False
    if falls:
        i = order.index(label)
        if i + 1 < len(order):
            succ.append(order[i + 1])
    return [s for s in succ if s in blocks]


def _following(blocks, order, label, index, budget, visit, seen=None):
    """Calls visit(inst, wait states already passed) for every instruction that can issue within
    `budget` wait states after position (label, index), over all control-flow successors."""
    seen = set() if seen is None else seen
    insts = blocks[label]
    passed = 0
    for inst in insts[index + 1:]:
        if passed >= budget:
            return
        visit(inst, passed)
        passed += inst.wait_states
    if passed < budget:
        for s in _successors(blocks, order, label):
            if (s, budget - passed) in seen:
                continue
            seen.add((s, budget - passed))
            _following(blocks, order, s, -1, budget - passed, lambda i, p, base=passed: visit(i, base + p), seen)


def lint_function(name, blocks, order):
    findings, dots = [], 0
    preds = {}
    for label in order:
        for s in _successors(blocks, order, label):
            preds.setdefault(s, []).append(label)

    def preceding(label, index, budget, visit, depth=0):
        passed = 0
        for inst in reversed(blocks[label][:index]):
            if passed >= budget:
                return
            visit(inst)
            passed += inst.wait_states
        if passed < budget and depth < 4:
            for p in preds.get(label, []):
                preceding(p, len(blocks[p]), budget - passed, visit, depth + 1)

    for label in order:
        for idx, inst in enumerate(blocks[label]):
            if inst.is_dpp and inst.is_valu and len(inst.operands) >= 2:
                src = _regs(inst.operands[1])

                def check_writer(prev, inst=inst, src=src):
                    hit = prev.vgpr_writes() & src
                    if hit:
                        findings.append({"rule": "valu-write-then-dpp-read", "function": name, "line": inst.line,
                                         "instruction": inst.text, "writer_line": prev.line, "writer": prev.text})
                preceding(label, idx, DPP_WAIT_STATES, check_writer)
            if inst.is_dot and inst.operands:
                dots += 1
                dst = _regs(inst.operands[0])

                def check_reader(nxt, passed, inst=inst, dst=dst):
                    if nxt.is_dot:
                        mult = set().union(*[_regs(o) for o in nxt.operands[1:3]]) if len(nxt.operands) > 2 else set()
                        if mult & dst:
                            findings.append({"rule": "dot-result-as-multiplicand", "function": name, "line": nxt.line,
                                             "instruction": nxt.text, "dot_line": inst.line})
                        return
                    if nxt.vgpr_reads() & dst:
                        findings.append({"rule": "dot-result-read-too-early", "function": name, "line": nxt.line,
                                         "instruction": nxt.text, "dot_line": inst.line, "wait_states": passed})
                    elif passed < DOT_OVERWRITE_WAIT_STATES and nxt.vgpr_writes() & dst:
                        findings.append({"rule": "dot-result-overwritten-too-early", "function": name, "line": nxt.line,
                                         "instruction": nxt.text, "dot_line": inst.line, "wait_states": passed})
                _following(blocks, order, label, idx, DOT_READ_WAIT_STATES, check_reader)
    return findings, dots


def lint_file(path):
    findings, dots, kernels = [], 0, 0
    for name, (blocks, order) in parse_functions(path).items():
        f, d = lint_function(name, blocks, order)
        findings += f
        dots += d
        kernels += 1 if d else 0
    return {"file": os.path.basename(path), "kernels_with_dots": kernels, "dot_instructions": dots, "findings": findings}


def main(argv):
    reports = [lint_file(p) for p in argv]
    print(json.dumps(reports, indent=1))
    return 1 if any(r["findings"] for r in reports) else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
