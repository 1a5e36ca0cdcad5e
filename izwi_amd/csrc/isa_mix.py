"""Static instruction mix of one kernel of a gfx950 assembly listing, by kind of instruction.

    hipcc $(HIPFLAGS) --cuda-device-only -S qmm_gemv_mfma.hip -o mfma.s      (`make isa-mix` does both steps)
    python3 isa_mix.py mfma.s <part of the kernel's mangled name> [ops]

For straight-line kernels (the single-stage batched decode forms) the static count is what a wave
executes, up to the short loops of the prologue and the k-split finish.  `ops` also lists the most
frequent opcodes.  The classes: 24-bit mul/mad = the integer scale products of the Q4_K block dots;
permlane swap = the in-register transposition of a panel into matrix-core operand order; bit ops =
nibble split, 6-bit scale unpacking, byte selects; convert + float = the f32 finish and the sum over
the k-split."""
import sys, re, collections
src, pat = sys.argv[1], sys.argv[2]
lines = open(src).read().split('\n')
start = None
for i, l in enumerate(lines):
    if re.match(r'^_Z\S*' + pat + r'\S*:', l): start = i; break
body = []
for l in lines[start + 1:]:
    if l.strip().startswith('s_endpgm'): break
    body.append(l)
cat = collections.Counter(); ops = collections.Counter()
def classify(op):
    if op.startswith('v_mfma'): return 'MFMA'
    if op.startswith('v_permlane'): return 'VALU permlane swap'
    if op.startswith('v_mad_i32_i24') or op.startswith('v_mad_u32_u24') or op.startswith('v_mul_i32_i24') or op.startswith('v_mul_u32_u24'): return 'VALU 24-bit mul/mad'
    if op.startswith('v_and') or op.startswith('v_lshr') or op.startswith('v_lshl') or op.startswith('v_bfe') or op.startswith('v_or') or op.startswith('v_bfi') or op.startswith('v_perm') or op.startswith('v_and_or') or op.startswith('v_lshl_or'): return 'VALU bit ops (and/shift/bfe/or)'
    if op.startswith('v_cvt'): return 'VALU convert'
    if op.startswith('v_fma') or op.startswith('v_mul_f32') or op.startswith('v_add_f32') or op.startswith('v_sub_f32') or op.startswith('v_fmac') or op.startswith('v_pk_'): return 'VALU float'
    if op.startswith('v_mov') or op.startswith('v_accvgpr'): return 'VALU mov'
    if op.startswith('v_add') or op.startswith('v_sub') or op.startswith('v_mul_lo') or op.startswith('v_mad_u64') or op.startswith('v_lshl_add') or op.startswith('v_add3') or op.startswith('v_mad'): return 'VALU int add/addr'
    if op.startswith('v_cmp') or op.startswith('v_cndmask'): return 'VALU cmp/select'
    if op.startswith('v_readfirstlane') or op.startswith('v_readlane'): return 'VALU readlane'
    if op.startswith('v_'): return 'VALU other'
    if op.startswith('ds_'): return 'LDS'
    if op.startswith('global_') or op.startswith('buffer_') or op.startswith('flat_') or op.startswith('scratch_'): return 'VMEM'
    if op.startswith('s_waitcnt'): return 's_waitcnt'
    if op.startswith('s_barrier'): return 's_barrier'
    if op.startswith('s_nop'): return 's_nop'
    if op.startswith('s_load') or op.startswith('s_buffer'): return 'SMEM'
    if op.startswith('s_cbranch') or op.startswith('s_branch'): return 'branch'
    if op.startswith('s_'): return 'SALU'
    return None
for l in body:
    t = l.strip()
    if not t or t.startswith(';') or t.startswith('.') or t.endswith(':'): continue
    op = t.split()[0]
    c = classify(op)
    if c is None: continue
    cat[c] += 1; ops[op] += 1
tot = sum(cat.values()); valu = sum(v for k, v in cat.items() if k.startswith('VALU'))
print(f"total {tot}  VALU(non-MFMA) {valu}  MFMA {cat['MFMA']}  VALU/MFMA {valu / max(cat['MFMA'],1):.2f}")
for k, v in sorted(cat.items(), key=lambda x: -x[1]): print(f"  {k:36s} {v}")
if len(sys.argv) > 3:
    for k, v in ops.most_common(40): print(f"     {k:28s} {v}")
