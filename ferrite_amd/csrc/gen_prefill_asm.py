"""Generates prefill_mainloop_asm.inc: the main loop of the 128-row expert GEMM kernels (gfx950) as one inline
assembly block with fixed registers.  Usage: python gen_prefill_asm.py prefill_mainloop_asm.inc

Per k step (128 k) a wave issues 32 scaled MFMAs (4 weight tiles x 8 row tiles of 16 unit rows) on a[0:127]; the
weights of its item arrive from global memory in v[64:159] (three buffers of a pair of k steps, loaded two pairs
ahead), the activations of the unit from a ring of six LDS stages that the block's four waves fill with
global -> LDS loads five steps ahead and read into v[160:223].  Everything that is not an MFMA is placed in the
shadow of one.  Loads complete in issue order and every step issues a fixed number of them, so the waits are counted
(the comments at each wait say what is behind it)."""
import sys

TAIL = 6                    # MFMAs at the end of each half step that carry no other instruction

NS = 6                      # ring stages (one k step of activations each, 16 KiB)
V_A = 64                    # v[64:159]  weights: 3 pair buffers x 2 steps x 4 tiles x 4 regs
V_B = 160                   # v[160:223] activations: 8 row tiles x 8 regs
V_BSC = 224                 # v[224:231] activation scale words, one per row tile
V_ASC = 232                 # v[232:235] weight scale words of the current group
V_ASCN = 236                # v[236:239] ... of the next group
OPSEL = {0: "op_sel_hi:[0,0,0]", 1: "op_sel:[1,1,0] op_sel_hi:[0,0,0]", 2: "op_sel_hi:[1,1,0]",
         3: "op_sel:[1,1,0] op_sel_hi:[1,1,0]"}

L = []
def e(s): L.append(s)

def a_regs(buf, half, t):           # 4 regs of tile t of step `half` of pair buffer `buf`
    b = V_A + buf * 32 + half * 16 + t * 4
    return f"v[{b}:{b+3}]"
def b_regs(tt):
    b = V_B + tt * 8
    return f"v[{b}:{b+7}]"
def acc(t, tt):
    b = (t * 8 + tt) * 4
    return f"a[{b}:{b+3}]"

def fill(stage):
    """the wave's quarter of the next k step of activations into ring stage `stage`; sources advance by 128 bytes
    while steps remain"""
    for j, off in enumerate(("%[bo0]", "%[bo1]", "%[bo2]", "%[bo3]")):
        e(f"s_add_u32 m0, %[ldsw], {stage * 16384 + j * 1024}")
        e("s_nop 0")
        e(f"global_load_lds_dwordx4 {off}, %[bbase]")
    e("s_cmp_gt_i32 %[nfill], 0")
    e("s_cselect_b32 %[t0], 128, 0")
    e("s_cselect_b32 %[t1], 1, 0")
    e("s_sub_u32 %[nfill], %[nfill], %[t1]")
    for off in ("%[bo0]", "%[bo1]", "%[bo2]", "%[bo3]"):
        e(f"v_add_u32_e32 {off}, %[t0], {off}")

def load_pair(buf):
    for half in range(2):
        for t in range(4):
            e(f"global_load_dwordx4 {a_regs(buf, half, t)}, %[wo{half}], %[wbase] offset:{t * 1024}")
    e("s_cmp_gt_i32 %[npair], 0")
    e("s_cselect_b32 %[t0], 8192, 0")
    e("s_cselect_b32 %[t1], 1, 0")
    e("s_sub_u32 %[npair], %[npair], %[t1]")
    e("v_add_u32_e32 %[wo0], %[t0], %[wo0]")
    e("v_add_u32_e32 %[wo1], %[t0], %[wo1]")

def load_scale(dst):
    e(f"global_load_dwordx4 v[{dst}:{dst+3}], %[wso], %[wsbase]")
    e("s_cmp_gt_i32 %[nsc], 0")
    e("s_cselect_b32 %[t0], 1024, 0")
    e("s_cselect_b32 %[t1], 1, 0")
    e("s_sub_u32 %[nsc], %[nsc], %[t1]")
    e("v_add_u32_e32 %[wso], %[t0], %[wso]")

def read_tiles(stage, first):
    base = "%[rd0]" if stage < 4 else "%[rd1]"
    soff = stage * 16384 if stage < 4 else stage * 16384 - 65536
    for tt in range(first, first + 4):
        b = V_B + tt * 8
        e(f"ds_read_b128 v[{b}:{b+3}], {base} offset:{soff + tt * 2048}")
        e(f"ds_read_b128 v[{b+4}:{b+7}], {base} offset:{soff + tt * 2048 + 1024}")

def mfma16(q, buf, half, first):
    for t in range(4):
        for tt in range(first, first + 4):
            e(f"v_mfma_scale_f32_16x16x128_f8f6f4 {acc(t, tt)}, {a_regs(buf, half, t)}, {b_regs(tt)}, {acc(t, tt)}, "
              f"v{V_ASC + t}, v{V_BSC + tt} {OPSEL[q]} cbsz:4")

def capture(fn, *args):
    """the lines fn(*args) would emit, as a list"""
    global L
    saved, L = L, []
    fn(*args)
    out, L = L, saved
    return out

def interleave(mfmas, fillers):
    """one wave per SIMD: whatever is not an MFMA goes into the shadow of one (an MFMA occupies the pipe for 32
    cycles; the wave issues in order), spread evenly"""
    n = len(mfmas) - TAIL          # the last MFMAs stay bare: they cover the latency of the last reads issued
    for i, m in enumerate(mfmas):
        e(m)
        if i < n:
            lo, hi = (len(fillers) * i) // n, (len(fillers) * (i + 1)) // n
            for f in fillers[lo:hi]:
                e(f)

def step(q, stage, buf, xstage=33):
    half = q & 1
    e(f"; ---- k step: q {q}, stage {stage}, pair buffer {buf}")
    if half == 0:
        e("s_waitcnt vmcnt(20)")                        # this pair's weights (and, for q 0, the scale word)
    if q == 0:
        for i in range(4):
            e(f"v_mov_b32_e32 v{V_ASC + i}, v{V_ASCN + i}")
        for tt in range(8):
            e(f"ds_read_b32 v{V_BSC + tt}, %[sc] offset:{tt * 256}")
        e("v_add_u32_e32 %[sc], 2048, %[sc]")
        e("s_waitcnt lgkmcnt(0)")
    f1 = capture(read_tiles, stage, 4) + capture(fill, (stage + NS - 1) % NS)
    if half == 0:
        f1 += capture(load_pair, (buf + 2) % 3)
    if q == 0:
        f1 += capture(load_scale, V_ASCN)
    interleave(capture(mfma16, q, buf, half, 0), f1)
    e("s_waitcnt lgkmcnt(0)")
    e(f"s_waitcnt vmcnt({xstage})")                     # own quarter of the next stage
    e("s_barrier")
    interleave(capture(mfma16, q, buf, half, 4), capture(read_tiles, (stage + 1) % NS, 0))
    e("s_waitcnt lgkmcnt(0)")

# ---- prologue: scale word, two pairs of weights, then the first five stages; what is issued first lands first, so
# vmcnt(16) (the four younger fills) leaves stage 0, the weights and the scale word complete
load_scale(V_ASCN)
load_pair(0)
load_pair(1)
for s_ in range(NS - 1):
    fill(s_)
for i in range(128):
    e(f"v_accvgpr_write_b32 a{i}, 0")
e("s_waitcnt vmcnt(16)")
e("s_barrier")
read_tiles(0, 0)
e("s_waitcnt lgkmcnt(0)")

def group(k0, peeled):
    for q in range(4):
        k = k0 + q
        # behind the fill of stage k+1 there are at least 33 younger loads from step 2 on, 25 in steps 0 and 1
        step(q, k % NS, (k // 2) % 3, 25 if (peeled and q < 2) else 33)
    e("s_sub_u32 %[grp], %[grp], 1")
    e("s_cmp_eq_u32 %[grp], 0")
    e("s_cbranch_scc1 2f")

group(0, True)
e("1:")
for k0 in (4, 8, 12):          # stages and pair buffers repeat every 12 steps
    group(k0, False)
e("s_branch 1b")
e("2:")
e("s_waitcnt vmcnt(0)")
e("s_nop 15")
e("s_nop 15")

out = []
out.append("// Generated by gen_prefill_asm.py: do not edit.  The main loop of the 128-row expert GEMM kernels as one")
out.append("// inline-assembly block with fixed registers: a[0:127] accumulators, v[64:159] weights (three buffers of a")
out.append("// pair of k steps), v[160:223] activation tiles, v[224:239] scale words.")
out.append("#define PR_MAINLOOP_ASM \\")
for ln in L:
    out.append('    "%s\\n\\t" \\' % ln)
out.append('    ""')
clob = [f'"v{i}"' for i in range(64, 240)] + [f'"a{i}"' for i in range(128)] + ['"vcc"', '"scc"', '"memory"']
out.append("#define PR_MAINLOOP_CLOBBERS \\")
for i in range(0, len(clob), 12):
    out.append("    " + ", ".join(clob[i:i + 12]) + ("," if i + 12 < len(clob) else "") + " \\")
out.append("")
open(sys.argv[1], "w").write("\n".join(out) + "\n")
print(len(L), "asm lines")
