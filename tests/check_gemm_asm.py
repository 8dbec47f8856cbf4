#!/usr/bin/env python3
"""Checks the generated assembly of the MFMA GEMM kernels for what the compiler cannot know.

The v_mfma_f32_32x32x16 instructions of lowbit_gemm.h sit in inline assembly, so the compiler neither knows
that their results arrive late (18 wait states for a 16-pass MFMA) nor that they are MFMAs at all.  The source
keeps every accumulator block in one place from the first MFMA to the epilogue; this script verifies that the
compiler went along with it, per kernel of an assembly listing (hipcc -S --cuda-device-only):

  1. every read of an accumulation register that an MFMA writes (v_accvgpr_read, the source of a v_accvgpr_mov,
     a store straight from accumulation registers) comes at least MIN_WAIT wait states after the nearest MFMA
     ahead of it in program order that writes that register - the compiler does move accumulator blocks between
     registers where variants of the main loop meet, which is harmless for a block whose MFMA is long done and
     loses a K step for the block written last;
  2. no such register is overwritten (v_accvgpr_mov, v_accvgpr_write) that soon after its MFMA either;
  3. the kernel uses no scratch memory and calls no function (a variant of the main loop that is not inlined
     keeps its closure in scratch and reads the weights with flat loads); kernels named after --allow-scratch may
     spill anywhere, kernels named after --allow-scratch-outside-loops only outside loops that hold MFMAs;
  4. no LDS-DMA takes its scalar base address from a v_readfirstlane less than 5 wait states earlier (VALU
     write of an SGPR followed by a VMEM read of it);
  5. no MFMA reads a vector register as its A or B operand that a VALU instruction wrote less than 2 wait states
     earlier (the kernels leave the wait states out where the operands are ready long before);
  6. a wait that leaves N loads in flight ahead of a workgroup barrier ("s_waitcnt vmcnt(N)", N > 0, then s_barrier:
     the step of the deep pipeline, whose youngest loads are the weights of two steps ahead) has at least N load
     instructions between the last LDS-DMA ahead of it and itself - loads retire in order, so with fewer (the
     compiler merged or dropped one) an LDS-DMA of x could still be in flight when the barrier publishes its buffer.
     A wait that the source marks with the comment "lowbit: this wait keeps the loads of one step in flight"
     (x two steps ahead as well) needs that many loads, LDS-DMAs included, since the barrier ahead of it.

usage: check_gemm_asm.py listing.s [--allow-scratch SUBSTRING ...] [--allow-scratch-outside-loops SUBSTRING ...]
Exit status 0 when every kernel passes, 1 otherwise.
"""
import re
import sys

MIN_WAIT = 18


def instructions(lines):
    for no, line in enumerate(lines):
        t = line.strip()
        if not t or t.startswith((";", ".", "//")) or t.endswith(":"):
            continue
        yield no, t


def wait_states(t):
    """Cycles an instruction keeps the wave busy at the least.  Another MFMA cannot issue before the one ahead of
    it has gone through its 8 passes of 4 cycles: whatever comes after a later MFMA is safe."""
    m = re.match(r"s_nop (\d+)", t)
    if m:
        return int(m.group(1)) + 1
    return 32 if t.startswith("v_mfma_f32_32x32x16") else 1


def regs(spec):
    """'a[4:7]' or 'a5' -> set of register numbers."""
    m = re.match(r"a\[(\d+):(\d+)\]", spec)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"a(\d+)$", spec)
    return {int(m.group(1))} if m else set()


def vregs(spec):
    """'v[4:7]' or 'v5' -> set of register numbers."""
    m = re.match(r"v\[(\d+):(\d+)\]", spec)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", spec)
    return {int(m.group(1))} if m else set()


def mfma_loops(lines):
    """Line numbers that lie inside an innermost loop holding an MFMA (a walk along K), from the loop comments the
    compiler puts behind block labels ('=>This Inner Loop Header', 'in Loop: Header=BB1_23', also on the '; %bb.N:'
    lines of blocks that are fallen into; a nested loop's header carries 'Parent Loop BB1_5' and its own
    'Loop Header' on the comment line below).  A loop around such loops - a workgroup that takes one tile after the
    other - is not one: what it holds besides them runs once per tile."""
    loop_of = {}                                   # line -> header name of the innermost loop it is in
    parents = set()
    current = None
    for no, line in enumerate(lines):
        t = line.strip()
        m = re.match(r"(?:\.L(BB\w+):|; %bb\.\d+:)(.*)", t)
        if m:
            rest = m.group(2)
            h = re.search(r"Header=(BB\w+)", rest)
            par = re.search(r"Parent Loop (BB\w+)", rest)
            if par:
                parents.add(par.group(1))
            below = lines[no + 1].strip() if no + 1 < len(lines) else ""
            if m.group(1) and ("Loop Header" in rest or (par and below.startswith(";") and "Loop Header" in below)):
                current = m.group(1)
            elif h:
                current = h.group(1)
            else:
                current = None
        elif t.startswith(";") and "Parent Loop" in t:
            par = re.search(r"Parent Loop (BB\w+)", t)
            if par:
                parents.add(par.group(1))
        if current:
            loop_of[no] = current
    with_mfma = {h for no, h in loop_of.items() if "v_mfma" in lines[no]} - parents
    return {no for no, h in loop_of.items() if h in with_mfma}


def check_kernel(name, lines, allow_scratch, first_line=0, allow_outside_loops=()):
    errors = []
    ins = [(no + first_line, t) for no, t in instructions(lines)]
    in_mfma_loop = {no + first_line for no in mfma_loops(lines)}
    scratch_seen = False
    mfma_dst = set()
    mfma_at = []
    for k, (no, t) in enumerate(ins):
        m = re.match(r"v_mfma_\S+ (a\[\d+:\d+\])", t)
        if m:
            mfma_dst |= regs(m.group(1))
            mfma_at.append(k)
    if not mfma_at:
        return errors
    mfma_writes = {}
    for k in mfma_at:
        mfma_writes[k] = regs(re.match(r"v_mfma_\S+ (a\[\d+:\d+\])", ins[k][1]).group(1))

    def since_write(k, wanted):
        """Wait states between the nearest MFMA ahead of instruction k (in program order, up to an unconditional
        branch) that writes one of `wanted` and instruction k; MIN_WAIT if there is none that close."""
        w = 0
        for j in range(k - 1, -1, -1):
            t = ins[j][1]
            if j in mfma_writes and (mfma_writes[j] & wanted):
                return w
            if re.match(r"s_branch|s_endpgm|s_setpc_b64", t):
                break
            w += wait_states(t)
            if w >= MIN_WAIT:
                break
        return MIN_WAIT

    for k, (no, t) in enumerate(ins):
        read = set()
        m = re.match(r"v_accvgpr_mov_b32 a\d+, (a\d+)", t)
        if m:
            read = regs(m.group(1))
        m = re.match(r"v_accvgpr_read_b32 v\d+, (a\d+)", t)
        if m:
            read = regs(m.group(1))
        m = re.match(r"(?:global|flat|scratch|buffer)_store\S* .*?(a\[\d+:\d+\]|a\d+)", t)
        if m:
            read = regs(m.group(1))
        if read & mfma_dst:
            w = since_write(k, read)
            if w < MIN_WAIT:
                errors.append(f"line {no + 1}: accumulator read {w} wait states after the MFMA that writes it: {t}")
        # overwriting a block while its MFMA is still in flight loses the result just the same
        m = re.match(r"v_accvgpr_(?:mov|write)_b32 (a\d+),", t)
        if m and (regs(m.group(1)) & mfma_dst):
            w = since_write(k, regs(m.group(1)))
            if w < MIN_WAIT:
                errors.append(f"line {no + 1}: accumulator overwritten {w} wait states after the MFMA that writes it: {t}")
        if re.match(r"s_swappc_b64|s_call_b64", t):
            errors.append(f"line {no + 1}: function call: {t}")
        if t.startswith("scratch_") and not any(a in name for a in allow_scratch):
            in_loop = no in in_mfma_loop
            if in_loop or not any(a in name for a in allow_outside_loops):
                if not scratch_seen or in_loop:
                    errors.append(f"line {no + 1}: scratch access{' inside an MFMA loop' if in_loop else ''}: {t}")
                scratch_seen = True
        m = re.match(r"v_mfma_\S+ a\[\d+:\d+\], (v\[\d+:\d+\]), (v\[\d+:\d+\])", t)
        if m:
            src = vregs(m.group(1)) | vregs(m.group(2))
            w = 0
            for j in range(k - 1, -1, -1):
                tj = ins[j][1]
                if tj.startswith("v_") and not tj.startswith("v_mfma"):
                    mm = re.match(r"\S+ (v\[\d+:\d+\]|v\d+)[, ]", tj + " ")
                    if mm and (vregs(mm.group(1)) & src):
                        errors.append(f"line {no + 1}: MFMA operand written by VALU {w} wait states earlier: {tj}")
                        break
                w += wait_states(tj)
                if w >= 2 or re.match(r"s_branch|s_cbranch|s_endpgm|s_setpc_b64", tj):
                    break
        m = re.match(r"s_waitcnt vmcnt\((\d+)\)$", t)
        if m and int(m.group(1)) > 0 and any(ins[j][1].startswith("s_barrier") for j in range(k + 1, min(k + 4, len(ins)))):
            whole_step = any("lowbit: this wait keeps the loads of one step in flight" in l
                             for l in lines[max(0, no - first_line - 8):no - first_line])
            younger, found = 0, False
            for j in range(k - 1, -1, -1):
                tj = ins[j][1]
                if tj.startswith("global_load_lds") and not whole_step:
                    found = True
                    break
                if re.match(r"(?:global|flat|scratch|buffer)_load", tj):
                    younger += 1
                if tj.startswith("s_barrier") and whole_step:
                    found = True
                    break
                if re.match(r"s_branch|s_cbranch|s_endpgm|s_setpc_b64|s_barrier", tj):
                    break
            if found and younger < int(m.group(1)):
                errors.append(f"line {no + 1}: {t} ahead of a barrier with only {younger} loads "
                              + ("since the barrier before it" if whole_step else "behind the last LDS-DMA"))
        m = re.match(r"global_load_lds_dwordx4 v\d+, s\[(\d+):(\d+)\]", t)
        if m:
            base = {int(m.group(1)), int(m.group(2))}
            w = 0
            for j in range(k - 1, -1, -1):
                mm = re.match(r"v_readfirstlane_b32 s(\d+),", ins[j][1])
                if mm and int(mm.group(1)) in base:
                    errors.append(f"line {no + 1}: LDS-DMA base written by VALU {w} wait states earlier")
                    break
                w += wait_states(ins[j][1])
                if w >= 5:
                    break
    return errors


def main(argv):
    if len(argv) < 2:
        print(__doc__)
        return 2
    allow, allow_outside = [], []
    if "--allow-scratch-outside-loops" in argv:
        i = argv.index("--allow-scratch-outside-loops")
        allow_outside = argv[i + 1:]
        argv = argv[:i]
    if "--allow-scratch" in argv:
        i = argv.index("--allow-scratch")
        allow = argv[i + 1:]
        argv = argv[:i]
    text = open(argv[1]).read().split("\n")
    starts = [i for i, l in enumerate(text) if re.match(r"_Z\w+:\s", l + " ")]
    bad = 0
    for n, s in enumerate(starts):
        name = text[s].split(":")[0]
        if "gemm_mfma_kernel" not in name and "gemm_ring_kernel" not in name:
            continue
        e = starts[n + 1] if n + 1 < len(starts) else len(text)
        errors = check_kernel(name, text[s:e], allow, s, allow_outside)
        label = "ok" if not errors else f"{len(errors)} problem(s)"
        print(f"{name}: {label}")
        for msg in errors[:10]:
            print("   ", msg)
        bad += bool(errors)
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
