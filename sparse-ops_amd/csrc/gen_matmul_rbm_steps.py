#!/usr/bin/env python3
"""Writes matmul_rbm_steps.inc: the step loop of the row-block-merged matmul kernel
(matmul_rbm.hip) as one inline-assembly string, SO_RBMM_STEPS_ASM.

    python3 gen_matmul_rbm_steps.py [matmul_rbm_steps.inc]

Why generated: a multiply-add's accumulator is chosen by VGPR index mode (M0 offsets the register
NUMBER), its X operand and its weight are fixed registers, so the loop body is straight-line code
whose shape is fixed by how many (row, weight) pairs each of the iteration's four columns has.
One body per shape ("class": 6 .. 16 pairs per column slot), unrolled over the four positions of
the operand rings; the kernel's stream lists the iterations class by class.

Registers (fixed):
  v[4:131]   the 128 accumulators of the wave's row block, v132 the spare one (padding pairs)
  v[134:149] X ring: 4 iterations x 4 column slots     v[150:165] weight ring: 4 iterations x 4
  v166 lane*4 (the lane's column inside a 64-column slab)   v167 (lane & 15) * 16
  s[2:7]   iterations per class, 16 bits each (classes 6 .. 16)
  s[8:11]  X as a buffer resource (base = the slab's first column, range = to the end of X)
  s[12:15] the wave's weight blocks as a buffer resource     s[16:17] the wave's records
  s18 byte offset of the current record (= of its weight block)
  s20 iterations left in the class - 1   s21 classes left   s22 the class the wave starts with
  s[24:27] byte offsets of the X rows of the iteration three ahead   s[32:63], s[64:95] accumulator indices of two iterations
A record (256 bytes) is one iteration: 32 dwords of accumulator indices (4 slots x 8 dwords x 2
halves, each 0xC000 | accumulator: M0's index-mode bits and offset), then the byte offsets of the 4 X
rows (row * pitch, written for the launch's pitch by a small kernel whenever the pitch changes); its 64
weights sit at the same offset of the weight array, slot-major.

Per iteration t (ring position t mod 4, index buffer t mod 2): X rows and weights of iteration
t + 3 are requested (buffer loads: an X row segment is one dword per lane, the weights one
dwordx4 per lane of each 16-lane row, replicated over the four rows so that DPP row_newbcast can
pick any of them), the indices of iteration t + 1 and the X rows of t + 4 by scalar loads; then
the multiply-adds of iteration t: M0 <- index (s_mov / s_lshr of a half), v_fmac_f32_dpp
acc[M0] += w(lane k of each row) * x.
"""
import sys

SLOTS, MAXP, ACC0, REC = 4, 16, 4, 256
CLASSES = list(range(6, 17))
DX = 4
LEAD = DX - 1
IBUF = [32, 64]
J = 24
XR = [134 + SLOTS * i for i in range(DX)]
WR = [150 + 4 * i for i in range(DX)]
LANE4, WLANE = 166, 167


def vmem(slot, jbase, off):
    o = []
    for k in range(SLOTS):
        o.append(f"buffer_load_dword v{XR[slot] + k}, v{LANE4}, s[8:11], s{jbase + k} offen")
    o.append(f"buffer_load_dwordx4 v[{WR[slot]}:{WR[slot] + 3}], v{WLANE}, s[12:15], s18 offen offset:{off}")
    return o


def top(t):
    o = vmem((t + LEAD) % DX, J, LEAD * REC)
    o.append(f"s_load_dwordx4 s[{J}:{J + 3}], s[16:17], s18 offset:{(LEAD + 1) * REC + 128}")
    nb = IBUF[(t + 1) % 2]
    o.append(f"s_load_dwordx16 s[{nb}:{nb + 15}], s[16:17], s18 offset:{REC}")
    o.append(f"s_load_dwordx16 s[{nb + 16}:{nb + 31}], s[16:17], s18 offset:{REC + 64}")
    o.append(f"s_add_u32 s18, s18, {REC}")
    o.append(f"s_waitcnt vmcnt({(SLOTS + 1) * LEAD})")
    return o


def fmas(t, s):
    o = []
    ib = IBUF[t % 2]
    for k in range(SLOTS):
        for p in range(s):
            w = k * s + p
            q, lam = w % 4, w // 4
            d = ib + 8 * k + p // 2
            o.append(f"s_mov_b32 m0, s{d}" if p % 2 == 0 else f"s_lshr_b32 m0, s{d}, 16")
            o.append(f"v_fmac_f32_dpp v{ACC0}, v{WR[t % DX] + q}, v{XR[t % DX] + k} row_newbcast:{lam} row_mask:0xf bank_mask:0xf")
    return o


def emit():
    o = []
    b1 = IBUF[1]
    # prologue: indices of iteration 0, X rows of iterations 0 .. 3; operands of iterations 0 .. 2 requested
    o.append(f"s_load_dwordx16 s[{IBUF[0]}:{IBUF[0] + 15}], s[16:17], s18 offset:0")
    o.append(f"s_load_dwordx16 s[{IBUF[0] + 16}:{IBUF[0] + 31}], s[16:17], s18 offset:64")
    for i in range(LEAD):
        o.append(f"s_load_dwordx4 s[{b1 + 4 * i}:{b1 + 4 * i + 3}], s[16:17], s18 offset:{i * REC + 128}")
    o.append(f"s_load_dwordx4 s[{J}:{J + 3}], s[16:17], s18 offset:{LEAD * REC + 128}")
    o.append("s_waitcnt lgkmcnt(0)")
    for i in range(LEAD):
        o += vmem(i, b1 + 4 * i, i * REC)
    o.append("s_set_gpr_idx_on 0, 0x0")
    for c in CLASSES:
        o.append(f"s_cmp_eq_u32 s22, {c}")
        o.append(f"s_cbranch_scc1 LD_{c}_0_%=")
    o.append("s_branch LDONE_%=")
    for ci, c in enumerate(CLASSES):
        nxt = CLASSES[(ci + 1) % len(CLASSES)]
        for a in range(DX):
            # enter class c with the rings at position a: done after all classes; skip an empty class
            o.append(f"LD_{c}_{a}_%=:")
            o.append("s_sub_u32 s21, s21, 1")
            o.append("s_cbranch_scc1 LDONE_%=")
            o.append(f"s_bfe_u32 s20, s{2 + ci // 2}, {hex(16 * (ci % 2) | (16 << 16))}")
            o.append("s_sub_u32 s20, s20, 1")
            o.append(f"s_cbranch_scc1 LD_{nxt}_{a}_%=")
            o.append(f"s_branch LB_{c}_{a}_%=")
        for a in range(DX):
            o.append(f"LB_{c}_{a}_%=:")
            o += top(a)
            o += fmas(a, c)
            o.append("s_waitcnt lgkmcnt(0)")
            o.append("s_sub_u32 s20, s20, 1")
            if a < DX - 1:
                o.append(f"s_cbranch_scc1 LD_{nxt}_{a + 1}_%=")
            else:
                o.append(f"s_cbranch_scc0 LB_{c}_0_%=")
                o.append(f"s_branch LD_{nxt}_0_%=")
    o.append("LDONE_%=:")
    o.append("s_waitcnt vmcnt(0) lgkmcnt(0)")
    o.append("s_mov_b32 m0, 0")
    o.append("s_set_gpr_idx_off")
    return o


def main():
    out = ["// generated by gen_matmul_rbm_steps.py -- do not edit", "#define SO_RBMM_STEPS_ASM \\"]
    for line in emit():
        sep = "\\n" if line.endswith(":") else "\\n\\t"
        out.append(f'    "{line}{sep}" \\')
    out.append('    ""')
    out.append("")
    open(sys.argv[1] if len(sys.argv) > 1 else "matmul_rbm_steps.inc", "w").write("\n".join(out))


if __name__ == "__main__":
    main()
