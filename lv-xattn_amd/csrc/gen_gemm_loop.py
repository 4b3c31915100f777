"""Writes the hand-scheduled main loop of the 256 x 256 bf16 GEMM tile (lvx_gemm.hip):

    python gen_gemm_loop.py bp > lvx_gemm_loop_bp.inc   (B stored [n][k]: 16-byte LDS reads)
    python gen_gemm_loop.py bt > lvx_gemm_loop_bt.inc   (B stored [k][n]: transposing LDS reads)

A is stored [m][k] in both.  One inline-asm statement runs a whole run of full 32-deep stages
(a multiple of four): request of the first three stages, then per stage the 16 MFMAs of a wave
(4 x 2 tiles of 32 x 32, two k-steps) with the LDS reads of the NEXT stage's twelve operands
and the wave's four global -> LDS loads of the stage three ahead placed between them, one
barrier per stage.  Operands are double-buffered in registers, so the MFMAs of a stage never
wait for LDS.  The loop keeps requesting after the last stage (the source pointers stop at it,
the copies land in buffers nobody reads any more) and keeps reading one stage past the end
(into registers nobody uses), so every trip is the same code.

Registers: v[0:127] accumulators acc[nt][mt] at 16 * (4 nt + mt)   v[128:175], v[176:223] the two
operand sets: A operands am[kk][mt] at +4 * (4 kk + mt), B operands bn[kk][nt] at +32 + 4 * (2 kk + nt)
v224, v225 A read addresses (k-step 0, 1) of stage buffer 0, v226, v227 the same + 64 KiB
v228, v229 B read addresses (bp: k-step 0, 1; bt: n tile 0, 1), v230, v231 the same + 64 KiB
v[232:235] global byte offsets of this wave's four 1 KiB chunks (two of A, two of B)
s[44:45] / s[46:47] A / B source of the next stage to request   s48 / s49 bytes per stage of A / B
s50 LDS address of this wave's chunk of stage buffer 0   s51 trips (stages / 4)   s52 stages still
to request   s53 .. s55 scratch
"""
import os
import sys

# experiment switches (comma separated in LVX_GEMM_OPTS); none is set in a normal build
OPTS = set(o for o in os.environ.get("LVX_GEMM_OPTS", "").split(",") if o)
BT = len(sys.argv) > 1 and sys.argv[1] == "bt"
MFMA = "v_mfma_f32_32x32x16_bf16"
STAGE, A_BYTES = 32768, 16384
SETS = (128, 176)


def vr(base, n=1):
    return f"v{base}" if n == 1 else f"v[{base}:{base + n - 1}]"


def am(s, kk, mt):
    return SETS[s] + 4 * (4 * kk + mt)


def bn(s, kk, nt):
    return SETS[s] + 32 + 4 * (2 * kk + nt)


def reads(slot, s):
    """LDS reads of the twelve operands of the stage in buffer `slot` into register set s, in the order
    the MFMAs want them."""
    hi = 2 if slot >= 2 else 0          # address registers of the upper 64 KiB
    off = (slot & 1) * STAGE
    out = []
    for kk in range(2):
        for nt in range(2):
            if BT:
                o = off + A_BYTES + kk * 8192
                out.append(f"ds_read_b64_tr_b16 {vr(bn(s, kk, nt), 2)}, v{228 + nt + hi} offset:{o}")
                out.append(f"ds_read_b64_tr_b16 {vr(bn(s, kk, nt) + 2, 2)}, v{228 + nt + hi} offset:{o + 2048}")
            else:
                out.append(f"ds_read_b128 {vr(bn(s, kk, nt), 4)}, v{228 + kk + hi} offset:{off + A_BYTES + nt * 2048}")
            if nt == 0:
                for mt in range(4):
                    out.append(f"ds_read_b128 {vr(am(s, kk, mt), 4)}, v{224 + kk + hi} offset:{off + mt * 2048}")
    return out


def request(slot):
    """This wave's four chunks of the next stage to request, into buffer `slot`; the sources move on unless
    they stand at the last stage."""
    base = slot * STAGE
    out = []
    for j in range(4):
        dst = base + (j * 8192 if j < 2 else A_BYTES + (j - 2) * 8192)
        out.append(f"s_add_i32 m0, s50, {dst}")
        out.append(f"global_load_lds_dwordx4 v{232 + j}, {'s[44:45]' if j < 2 else 's[46:47]'}")
    out += ["s_cmp_gt_u32 s52, 1", "s_cselect_b32 s53, s48, 0", "s_cselect_b32 s54, s49, 0", "s_cselect_b32 s55, 1, 0",
            "s_add_u32 s44, s44, s53", "s_addc_u32 s45, s45, 0", "s_add_u32 s46, s46, s54", "s_addc_u32 s47, s47, 0",
            "s_sub_u32 s52, s52, s55"]
    return out


def stage(u):
    """Stage s with s % 4 == u: its MFMAs from set u & 1, the reads of stage s+1, the request of stage s+3."""
    cur, nxt = u & 1, (u + 1) & 1
    out = ["s_waitcnt vmcnt(4)", "s_waitcnt lgkmcnt(0)", "s_barrier"]
    rd = reads((u + 1) % 4, nxt)
    rq = request((u + 3) % 4)
    n_reads = len(rd)
    k = 0
    for kk in range(2):
        for nt in range(2):
            for mt in range(4):
                a = 16 * (4 * nt + mt)
                out.append(f"{MFMA} {vr(a, 16)}, {vr(bn(cur, kk, nt), 4)}, {vr(am(cur, kk, mt), 4)}, {vr(a, 16)}")
                # one or two LDS reads behind every MFMA, the request spread over the second half
                n_rd = (n_reads * (k + 1)) // 12 - (n_reads * k) // 12 if k < 12 else 0
                for _ in range(n_rd):
                    out.append(rd.pop(0))
                if 8 <= k < 12:         # an m0 write and its load
                    out.append(rq.pop(0))
                    out.append(rq.pop(0))
                elif k >= 12:           # where the next request reads from
                    for _ in range(3 if k < 15 else len(rq)):
                        if rq:
                            out.append(rq.pop(0))
                k += 1
    out += rd + rq
    return out


def main():
    pro = []
    for slot in range(3):
        pro += request(slot)
    pro += ["s_waitcnt vmcnt(8)", "s_barrier"] + reads(0, 0)
    body = []
    for u in range(4):
        body += stage(u)
    lines = pro + ["LVX_GEMM_LOOP_%=:"] + body + ["s_sub_u32 s51, s51, 1", "s_cmp_lg_u32 s51, 0", "s_cbranch_scc1 LVX_GEMM_LOOP_%=",
                                                  "s_waitcnt vmcnt(0)", "s_waitcnt lgkmcnt(0)", "s_barrier", "s_nop 15", "s_nop 3"]
    print("// generated by gen_gemm_loop.py - do not edit")
    if "nodma" in OPTS:
        lines = [l for l in lines if not l.startswith("global_load_lds") and not l.startswith("s_add_i32 m0")]
    if "nolds" in OPTS:
        lines = [l for l in lines if not l.startswith("ds_read")]
    if "nobar" in OPTS:
        lines = [l for l in lines if l != "s_barrier"]
    if "nomfma" in OPTS:
        lines = [l for l in lines if not l.startswith("v_mfma")]
    for l in lines:
        print(f'"{l}\\n"')


main()
