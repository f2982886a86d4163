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
