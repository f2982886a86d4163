"""Build-time checks of the tile kernels' generated assembly.

check(): the block-scaled GEMM kernel.

That kernel loads its block scales with an inline-assembly buffer load whose result the compiler
believes to be available at once, although it arrives later (the kernel waits for it by counting
vector-memory instructions).  This is only sound if the compiler never touches the destination
registers between the load and the scaled MFMAs that consume them: a copy made in between would
read the registers before the data has landed.  The check walks each such kernel's instruction
stream and fails if
  * any instruction other than a scaled MFMA reads a register last written by such a load, or
  * a scaled MFMA takes a scale from a register last written by anything else.

check_lds_base(): see there.
"""
import re
import sys

KERNEL = re.compile(r'^(_ZN\S*gemm_tn_tile_ringINS_6MxE4M3\S*):[^\n]*\n(.*?)\n\s*\.Lfunc_end', re.S | re.M)
SCALED_MFMA = "v_mfma_scale_f32_16x16x128_f8f6f4"
ASYNC_LOAD = "buffer_load_dwordx2"
NO_DESTINATION = ("buffer_store", "ds_write", "global_store", "s_", "v_cmp", "v_cmpx")


def _vgprs(text):
    out = set()
    for a, b in re.findall(r'\bv\[(\d+):(\d+)\]', text):
        out.update(range(int(a), int(b) + 1))
    for a in re.findall(r'\bv(\d+)\b', text):
        out.add(int(a))
    return out


def check(asm_path):
    """Returns the number of scale operands checked; raises RuntimeError on a violation."""
    src = open(asm_path).read()
    kernels = KERNEL.findall(src)
    if not kernels:
        raise RuntimeError("no block-scaled kernel found in " + asm_path)
    total = 0
    for name, body in kernels:
        lines = [l.split(';')[0].strip() for l in body.split('\n')]
        state = {}
        reads = 0
        for l in lines:
            if not l or l.startswith('.') or l.endswith(':'):
                continue
            parts = l.split(None, 1)
            if len(parts) < 2:
                continue
            op, rest = parts
            ops = [o.strip() for o in rest.split(',')]
            no_dst = op.startswith(NO_DESTINATION)
            dst = set() if no_dst else _vgprs(ops[0])
            if op == SCALED_MFMA:
                for r in _vgprs(ops[4]) | _vgprs(ops[5].split()[0]):
                    reads += 1
                    if state.get(r) != 'loaded':
                        raise RuntimeError("%s: scale operand v%d is not fresh from a scale load: %s" % (name, r, l))
                if any(state.get(r) == 'loaded' for r in _vgprs(','.join(ops[1:4]))):
                    raise RuntimeError("%s: a scale register is used as a data operand: %s" % (name, l))
            else:
                for r in _vgprs(','.join(ops if no_dst else ops[1:])):
                    if state.get(r) == 'loaded':
                        raise RuntimeError("%s: v%d is read while it belongs to a scale load: %s" % (name, r, l))
            for r in dst:
                state[r] = 'loaded' if op == ASYNC_LOAD else 'other'
        if reads == 0:
            raise RuntimeError(name + ": no scaled MFMA found")
        total += reads
    return total


RING_KERNEL = re.compile(r'^(_ZN\S*gemm_tn_tile_ring\S*):[^\n]*\n(.*?)\n\s*\.Lfunc_end', re.S | re.M)


def check_lds_base(asm_path):
    """The tile kernels write the LDS base of a direct-to-LDS copy to M0 up to one MFMA before the
    copy is issued, in a separate inline-assembly statement.  That is only sound if nothing else
    writes M0 in these kernels and every copy has its own write: in each kernel the writes of M0
    must all be the kernel's own `s_add_u32 m0, ...` and must alternate one to one with the
    `buffer_load_dwordx4 ... lds` instructions.  Returns the number of copies checked."""
    src = open(asm_path).read()
    kernels = RING_KERNEL.findall(src)
    if not kernels:
        raise RuntimeError("no tile kernel found in " + asm_path)
    total = 0
    for name, body in kernels:
        armed = False
        for l in (x.split(';')[0].strip() for x in body.split('\n')):
            if not l:
                continue
            parts = l.split(None, 1)
            ops = parts[1] if len(parts) > 1 else ""
            first = ops.split(',')[0].strip()
            if first == "m0":
                if not l.startswith("s_add_u32 m0,"):
                    raise RuntimeError("%s: M0 is written by something else than the copy set-up: %s" % (name, l))
                if armed:
                    raise RuntimeError("%s: two writes of M0 without a copy in between: %s" % (name, l))
                armed = True
            elif parts[0] == "buffer_load_dwordx4" and ops.rstrip().endswith("lds"):
                if not armed:
                    raise RuntimeError("%s: a direct-to-LDS copy without its own write of M0: %s" % (name, l))
                armed = False
                total += 1
        if armed:
            raise RuntimeError(name + ": a write of M0 that no copy uses")
    if total == 0:
        raise RuntimeError("no direct-to-LDS copy found in " + asm_path)
    return total


if __name__ == "__main__":
    print("scale operands checked:", check(sys.argv[1]))


# ---------------------------------------------------------------------------------------------
# Distances the hardware wants and the compiler cannot (or does not) enforce.
#
# Rule 1, wide stores.  A vector-memory store of more than 8 bytes per lane reads its data registers
# over several cycles after it has issued; the ISA therefore asks for idle wait states between such a
# store and the next write of a register that holds its data.  The compiler inserts them only for
# stores without a scalar offset register, and the tile kernels' stores have one; with nothing but the
# two wait states the compiler adds elsewhere, a few lanes of a store's first data register were seen
# to carry the NEXT store's value.  The kernels therefore keep every store's data registers untouched
# while the following block is converted (tile_store.h), and this check holds them to it: on every
# path, no instruction within STORE_DATA_WINDOW wait states after a store of 8 bytes or more per
# lane may write a register the store reads as data.
#
# Rule 2, matrix-core results.  The MFMAs of the 256-row tile kernels, of the block-scaled kernels
# and of the calibration kernel are inline assembly, so the compiler does not know that their
# results arrive up to 16 passes later and inserts no wait states in front of the first reader
# (for MFMAs it emits itself it does, from the true pass count; those are not checked here).
# On every path, no instruction other than an MFMA that accumulates in place into exactly the same
# registers may touch an MFMA's destination within MFMA_RESULT_WINDOW wait states (16 passes + 3,
# the ISA's figure for the longest MFMA; the ones used here take 4 or 8 passes).
#
# A wait state is one issued instruction; s_nop N counts N + 1.
STORE_DATA_WINDOW = 12
MFMA_RESULT_WINDOW = 19

ANY_KERNEL = re.compile(r'^(_Z\w+):[^\n]*\n(.*?)\n\s*\.Lfunc_end', re.S | re.M)
_WIDE_STORE = re.compile(r'^(buffer|global|flat|scratch)_store_(dwordx[234]|b64|b96|b128)$')
_LABEL = re.compile(r'^([.\w$]+):')
_WRITES_TWO = ("v_permlane16_swap", "v_permlane32_swap", "v_swap_b32")
_NO_VECTOR_DST = ("buffer_store", "global_store", "flat_store", "scratch_store", "ds_write", "ds_store", "s_", "v_cmp",
                  "v_cmpx", "v_readlane", "v_readfirstlane", "buffer_wbl2", "buffer_inv", "buffer_atomic", "global_atomic")


def _regs(text, bank):
    """Register numbers of bank 'v' or 'a' named in an operand string."""
    out = set()
    for a, b in re.findall(r'\b%s\[(\d+):(\d+)\]' % bank, text):
        out.update(range(int(a), int(b) + 1))
    for a in re.findall(r'\b%s(\d+)\b' % bank, text):
        out.add(int(a))
    return out


class _Inst:
    __slots__ = ("op", "ops", "text", "writes", "reads", "wait", "inline")

    def __init__(self, text, inline=False):
        self.text = text
        self.inline = inline                  # part of an inline-assembly statement
        parts = text.split(None, 1)
        self.op = parts[0]
        self.ops = [o.strip() for o in parts[1].split(',')] if len(parts) > 1 else []
        self.wait = 1
        if self.op == "s_nop" and self.ops:
            self.wait = int(self.ops[0], 0) + 1
        n_dst = 0
        if self.ops and not self.op.startswith(_NO_VECTOR_DST):
            n_dst = 2 if self.op.startswith(_WRITES_TWO) else 1
            if self.ops[-1].split()[-1] == "lds" and self.op.startswith("buffer_load"):
                n_dst = 0                     # direct-to-LDS copy: the first operand is the address
        dst = ','.join(self.ops[:n_dst])
        src = ','.join(self.ops if n_dst == 0 else (self.ops if self.op.startswith(_WRITES_TWO) else self.ops[n_dst:]))
        self.writes = {('v', r) for r in _regs(dst, 'v')} | {('a', r) for r in _regs(dst, 'a')}
        self.reads = {('v', r) for r in _regs(src, 'v')} | {('a', r) for r in _regs(src, 'a')}


def _parse(body):
    """-> (instructions, label -> index of the instruction that follows it)."""
    insts, labels = [], {}
    inline = False
    for raw in body.split('\n'):
        if "#ASMSTART" in raw:
            inline = True
        elif "#ASMEND" in raw:
            inline = False
        l = raw.split(';')[0].strip()
        if not l or l.startswith('.') and not _LABEL.match(l):
            continue
        m = _LABEL.match(l)
        if m:
            labels[m.group(1)] = len(insts)
            continue
        insts.append(_Inst(l, inline))
    return insts, labels


def _window(insts, labels, start, limit):
    """Instructions reachable from the one after `start` within `limit` wait states, on any path:
    yields (index, wait states issued between insts[start] and it)."""
    seen = {}
    todo = [(start + 1, 0)]
    while todo:
        i, d = todo.pop()
        while i < len(insts) and d < limit:
            if seen.get(i, limit + 1) <= d:
                break
            seen[i] = d
            ins = insts[i]
            yield i, d
            d += ins.wait
            if ins.op == "s_endpgm":
                break
            if ins.op in ("s_setpc_b64", "s_swappc_b64"):
                raise RuntimeError("indirect jump inside a checked window: " + ins.text)
            if ins.op == "s_branch":
                i = labels[ins.ops[0]]
                continue
            if ins.op.startswith("s_cbranch"):
                todo.append((labels[ins.ops[0]], d))
            i += 1


def check_hazard_distances(asm_path, kernel_filter=None):
    """Rules 1 and 2 above on every kernel of the file whose mangled name contains kernel_filter.
    Returns (stores checked, MFMAs checked); raises RuntimeError on a violation."""
    src = open(asm_path).read()
    stores = mfmas = 0
    found = False
    for name, body in ANY_KERNEL.findall(src):
        if kernel_filter and kernel_filter not in name:
            continue
        found = True
        insts, labels = _parse(body)
        for i, ins in enumerate(insts):
            if _WIDE_STORE.match(ins.op):
                operand = ins.ops[0] if ins.op.startswith("buffer_") else ins.ops[1]   # global/flat: address first
                data = {('v', r) for r in _regs(operand, 'v')} | {('a', r) for r in _regs(operand, 'a')}
                stores += 1
                for j, d in _window(insts, labels, i, STORE_DATA_WINDOW):
                    hit = insts[j].writes & data
                    if hit:
                        raise RuntimeError("%s: %s rewrites data of `%s` after %d wait states (need %d)"
                                           % (name, insts[j].text, ins.text, d, STORE_DATA_WINDOW))
            elif ins.inline and (ins.op.startswith("v_mfma") or ins.op.startswith("v_smfmac")):
                mfmas += 1
                dst = ins.writes
                for j, d in _window(insts, labels, i, MFMA_RESULT_WINDOW):
                    other = insts[j]
                    if not ((other.reads | other.writes) & dst):
                        continue
                    in_place = other.op.startswith("v_mfma") and other.writes == dst and \
                        other.op == ins.op and len(other.ops) > 3 and other.ops[0].split()[0] == other.ops[3].split()[0] and \
                        not ({('v', r) for r in _regs(','.join(other.ops[1:3]), 'v')} |
                             {('a', r) for r in _regs(','.join(other.ops[1:3]), 'a')}) & dst
                    if not in_place:
                        raise RuntimeError("%s: `%s` touches the result of `%s` after %d wait states (need %d)"
                                           % (name, other.text, ins.text, d, MFMA_RESULT_WINDOW))
    if not found:
        raise RuntimeError("no kernel matching %r in %s" % (kernel_filter, asm_path))
    return stores, mfmas


def check_no_scratch(asm_path):
    """The ring kernels count the vector-memory instructions in flight by hand (s_waitcnt vmcnt(N) with N
    derived from the copies they issue); a register spill would add loads and stores of its own to
    that count.  No kernel of the file may use scratch memory or spill a vector register.  Returns
    the number of kernels checked."""
    src = open(asm_path).read()
    sizes = [int(x) for x in re.findall(r'^\s*\.private_segment_fixed_size:\s*(\d+)', src, re.M)]
    spills = [int(x) for x in re.findall(r'^\s*\.vgpr_spill_count:\s*(\d+)', src, re.M)]
    if not sizes or len(sizes) != len(spills):
        raise RuntimeError("no kernel metadata found in " + asm_path)
    if any(sizes) or any(spills):
        raise RuntimeError("%s: a kernel uses scratch memory (bytes per lane %r, spilled registers %r)"
                           % (asm_path, sizes, spills))
    return len(sizes)
