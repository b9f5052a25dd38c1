"""Static check of the device assembly for the hand-issued register loads.

Some tile kernels issue global loads that land in VGPRs from inline asm, so that they share the hand-counted
vmcnt scheme of the direct-to-LDS loads.  The compiler believes such a destination register holds its value
as soon as the asm statement has been issued; the code is only correct while nothing reads, copies, spills or
overwrites that register before an `s_waitcnt vmcnt(n)` that really covers the load.  This module proves that
property on the generated assembly, for every path of the control-flow graph:

  for every vector-memory load between `;;#ASMSTART` / `;;#ASMEND` whose destination is a VGPR (not an LDS
  load), on every path from the load: no instruction names a destination register until an `s_waitcnt` whose
  vmcnt is <= the number of vector-memory loads issued after the load on that path (loads return in order
  among themselves, so the load has then landed; stores are not counted, they may complete at any time).

It also refuses register spills and a private (scratch) segment, in every kernel of the file: with hand-issued loads
a spill breaks the code, without them it costs a tile kernel several times its run time and nothing else reports it.

A second property concerns the scalar registers such an instruction reads (its base address).  A vector-memory
instruction needs five wait states after a VALU instruction (v_readfirstlane_b32, v_readlane_b32, a compare or a
carry-out) wrote a scalar register it reads; the hardware does not interlock.  The compiler inserts the wait
states for the instructions it emits and cannot see into an asm statement, so:

  for every VALU instruction that writes scalar registers, on every path of fewer than five wait states from it
  (an instruction is one wait state, `s_nop n` is n + 1): no vector-memory instruction between `;;#ASMSTART` /
  `;;#ASMEND` reads one of those registers.

Likewise a direct-to-LDS load reads M0 (its LDS base) and needs one wait state after a scalar write to M0: an
asm `..._lds_...` load must not come right after the instruction that writes m0.

build.py runs these checks on every source and fails the build when one does not hold.
"""
import re
import sys

_LABEL = re.compile(r"^([.\w$]+):")
_REG1 = re.compile(r"\bv(\d+)\b")
_REGR = re.compile(r"\bv\[(\d+):(\d+)\]")
_VMCNT = re.compile(r"vmcnt\((\d+)\)")
# Only loads count as "younger": loads return in order among themselves, while a store may be acknowledged
# before or after the loads around it, so a pending store can never vouch for a load having landed.
_VM_PREFIX = ("global_load", "buffer_load", "flat_load", "scratch_load")


def _regs(text):
    out = set(int(m) for m in _REG1.findall(text))
    for a, b in _REGR.findall(text):
        out.update(range(int(a), int(b) + 1))
    return out


class _Func:
    def __init__(self, name):
        self.name = name
        self.ins = []          # (opcode, operand text, in_asm_block)
        self.labels = {}       # label -> index of the next instruction


def _parse(path):
    funcs, cur, in_asm = [], None, False
    meta = {}                  # kernel name -> {"spill": n, "private": n}
    meta_name = None
    for raw in open(path, errors="replace"):
        line = raw.split("//")[0].rstrip()
        s = line.strip()
        if s.startswith("- ."):                  # first key of a YAML list item in the kernel metadata
            s = s[2:]
        if s.startswith(".name:"):
            meta_name = s.split(":", 1)[1].strip()
            meta.setdefault(meta_name, {})
        elif meta_name and s.startswith(".vgpr_spill_count:"):
            meta[meta_name]["spill"] = int(s.split(":")[1])
        elif meta_name and s.startswith(".sgpr_spill_count:"):
            meta[meta_name]["sspill"] = int(s.split(":")[1])
        elif meta_name and s.startswith(".private_segment_fixed_size:"):
            meta[meta_name]["private"] = int(s.split(":")[1])
        if s.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if s.startswith(";;#ASMEND"):
            in_asm = False
            continue
        m = _LABEL.match(line)
        if m and not line[0].isspace():
            lab = m.group(1)
            if not lab.startswith(".L"):
                cur = _Func(lab)
                funcs.append(cur)
            elif cur is not None:
                cur.labels[lab] = len(cur.ins)
            continue
        if cur is None or not s or s.startswith(".") or s.startswith(";"):
            continue
        code = s.split(";")[0].strip()
        if not code:
            continue
        parts = code.split(None, 1)
        cur.ins.append((parts[0], parts[1] if len(parts) > 1 else "", in_asm))
    return funcs, meta


def _is_vm(op):
    return op.startswith(_VM_PREFIX)


_SREG1 = re.compile(r"\bs(\d+)\b")
_SREGR = re.compile(r"\bs\[(\d+):(\d+)\]")
_VM_ANY = ("global_", "buffer_", "flat_", "scratch_")
_VALU_SGPR_WAIT_STATES = 5
# VALU instructions whose SECOND operand is a scalar destination (carry-out / scale flag)
_SDST_SECOND = ("v_mad_u64_u32", "v_mad_i64_i32", "v_add_co_u32", "v_sub_co_u32", "v_subrev_co_u32", "v_addc_co_u32",
                "v_subb_co_u32", "v_subbrev_co_u32", "v_div_scale_f32", "v_div_scale_f64")


def _sregs(text):
    out = set("s%d" % int(m) for m in _SREG1.findall(text))
    for a, b in _SREGR.findall(text):
        out.update("s%d" % i for i in range(int(a), int(b) + 1))
    if re.search(r"\bvcc\b", text):
        out.update(("vcc_lo", "vcc_hi"))
    out.update(re.findall(r"\bvcc_(?:lo|hi)\b", text))
    return out


def _valu_sgpr_writes(op, args):
    """Scalar registers a VALU instruction writes (empty for everything else)."""
    if not op.startswith("v_"):
        return set()
    ops = [a.strip() for a in args.split(",")]
    out = set()
    if ops and not ops[0].startswith(("v", "a")):
        out |= _sregs(ops[0])
    if op.startswith(_SDST_SECOND) and len(ops) > 1:
        out |= _sregs(ops[1])
    return out


def _check_scalar_settle(f, problems):
    """No asm vector-memory instruction reads a scalar register within five wait states of a VALU write to it."""
    checked = 0
    for i in range(1, len(f.ins)):
        op, args, in_asm = f.ins[i]
        pop, pargs, _ = f.ins[i - 1]
        if in_asm and op.startswith(_VM_ANY) and "_lds_" in op and pop.startswith("s_") and \
                pargs.split(",")[0].strip() == "m0":
            problems.append("%s: asm `%s %s` reads M0 with no wait state after `%s %s`" % (f.name, op, args, pop, pargs))
    for wi, (op, args, _) in enumerate(f.ins):
        written = _valu_sgpr_writes(op, args)
        if not written:
            continue
        seen = {}
        stack = [(wi + 1, _VALU_SGPR_WAIT_STATES, frozenset(written))]
        while stack:
            i, left, live = stack.pop()
            while left > 0 and live and i < len(f.ins):
                if seen.get((i, live), 0) >= left:
                    break
                seen[(i, live)] = left
                op2, args2, in_asm = f.ins[i]
                if in_asm and op2.startswith(_VM_ANY):
                    checked += 1
                    hit = live & _sregs(args2)
                    if hit:
                        problems.append("%s: asm `%s %s` reads %s only %d wait states after `%s %s` wrote it (needs %d)"
                                        % (f.name, op2, args2, sorted(hit), _VALU_SGPR_WAIT_STATES - left, op, args,
                                           _VALU_SGPR_WAIT_STATES))
                        break
                if op2 == "s_endpgm":
                    break
                if op2.startswith("s_") and not op2.startswith(("s_cbranch", "s_branch", "s_nop", "s_waitcnt", "s_cmp",
                                                                 "s_bitcmp", "s_barrier")):
                    # a scalar-ALU or scalar-memory write replaces the VALU's value: interlocked from here on
                    live = live - _sregs(args2.split(",")[0])
                left -= (int(args2.strip() or 0) + 1) if op2 == "s_nop" else 1
                if op2 == "s_branch":
                    i = f.labels.get(args2.strip(), len(f.ins))
                    continue
                if op2.startswith("s_cbranch"):
                    tgt = f.labels.get(args2.strip())
                    if tgt is not None:
                        stack.append((tgt, left, live))
                i += 1
    return checked


def check_file(path):
    """Returns (number of hand-issued register loads checked, list of violation strings)."""
    funcs, meta = _parse(path)
    problems, checked = [], 0
    with_loads = set()
    for f in funcs:
        if any(in_asm and op.startswith(("global_load", "buffer_load", "flat_load")) and "_lds_" not in op for op, _, in_asm in f.ins):
            with_loads.add(f.name)
    # No kernel of the library is meant to spill: a tile kernel that does still gives right results, several times
    # slower (a lane predicate around one load in the K loop of the 256-column kernel cost 450 bytes of scratch and a
    # factor of eight), and nothing else would say so.
    for name, md in meta.items():
        if name not in with_loads and (md.get("spill", 0) or md.get("private", 0)):
            problems.append("%s: kernel has %d spilled VGPRs and %d bytes of scratch" % (name, md.get("spill", 0), md.get("private", 0)))
    for f in funcs:
        if any(in_asm and op.startswith(_VM_ANY) for op, _, in_asm in f.ins):
            _check_scalar_settle(f, problems)
        loads = [i for i, (op, args, in_asm) in enumerate(f.ins)
                 if in_asm and op.startswith(("global_load", "buffer_load", "flat_load")) and "_lds_" not in op]
        if not loads:
            continue
        md = meta.get(f.name, {})
        if md.get("spill", 0) or md.get("private", 0):
            problems.append("%s: kernel with hand-issued register loads has %d spilled VGPRs and %d bytes of scratch"
                            % (f.name, md.get("spill", 0), md.get("private", 0)))
        for li in loads:
            checked += 1
            dest = _regs(f.ins[li][1].split(",")[0])
            if not dest:
                problems.append("%s: cannot parse the destination of `%s %s`" % (f.name, *f.ins[li][:2]))
                continue
            best = {}                      # instruction index -> fewest younger vector-memory instructions seen
            stack = [(li + 1, 0)]
            while stack:
                i, younger = stack.pop()
                while True:
                    if i >= len(f.ins):
                        problems.append("%s: load at #%d: ran off the function without a covering s_waitcnt" % (f.name, li))
                        break
                    if i in best and best[i] <= younger:
                        break
                    best[i] = younger
                    op, args, _ = f.ins[i]
                    if op == "s_waitcnt":
                        m = _VMCNT.search(args)
                        if m and int(m.group(1)) <= younger:
                            break                                   # the load has landed on this path
                    elif op == "s_endpgm":
                        break                                       # never consumed on this path
                    if op != "s_waitcnt" and dest & _regs(args):
                        problems.append("%s: `%s %s` touches v%s of the hand-issued load #%d (`%s`) before a covering "
                                        "s_waitcnt" % (f.name, op, args, sorted(dest & _regs(args)), li, f.ins[li][1]))
                        break
                    if _is_vm(op):
                        younger += 1
                    if op == "s_branch":
                        i = f.labels.get(args.strip(), len(f.ins))
                        continue
                    if op.startswith("s_cbranch"):
                        tgt = f.labels.get(args.strip())
                        if tgt is not None:
                            stack.append((tgt, younger))
                    if op in ("s_setpc_b64", "s_swappc_b64"):
                        problems.append("%s: indirect jump after a hand-issued load" % f.name)
                        break
                    i += 1
    return checked, problems


if __name__ == "__main__":
    total, bad = 0, []
    for p in sys.argv[1:]:
        n, pr = check_file(p)
        total += n
        bad += pr
    print("%d hand-issued register loads checked, %d problems" % (total, len(bad)))
    for b in bad[:40]:
        print("  " + b)
    sys.exit(1 if bad else 0)
