"""Writes lvx_fwd_loop_wide.inc: the hand-scheduled steady-state loop of the forward kernel whose
waves own TWO blocks of 32 text rows (lvx_fwd.hip, fwd_kernel_wide).

    python gen_fwd_loop_wide.py > lvx_fwd_loop_wide.inc

Same pipeline as gen_fwd_loop.py - per key tile t the MFMAs of S(t+1) = K(t+1) Q^T and of
O += V(t)^T P(t) in program order, with the exponentials of tile t, the row maximum of tile t+1,
the LDS operand reads and the global -> LDS loads between them - but every K or V operand read
from LDS feeds two MFMAs, one per row block, so a wave reads half as many LDS bytes and a
work-group requests half as many tile bytes per MFMA.  The wave has the SIMD to itself (512
registers): the O^T accumulators and Q^T live in accumulation registers, which only MFMAs touch
(the rare rescale of O goes through a few VGPRs).

The statement receives O^T and Q^T in VGPRs, moves them up at entry and back at exit, and uses
the VGPRs they arrived in for scores, P and operand slots in between.

Register map (must match the constraints of the asm statement in lvx_fwd.hip), b = row block:
  at entry / exit: v[64 b : 64 b + 63] O^T of block b, v[128 + 32 b : 159 + 32 b] Q^T of block b
  inside: a[64 b : 64 b + 63] O^T, a[128 + 32 b : 159 + 32 b] Q^T
          v[64 b : 64 b + 31] scores set A, v[64 b + 32 : 64 b + 63] scores set B
          v[128 + 16 b : 143 + 16 b] P^T   v[160:199] ten operand slots
  v[200:207] K read addresses (per k-step)   v[208:215] V read addresses (d tile x half)
  v[216:219] global offsets of the 4 row groups   v220+b m   v222+b l   v224+b alpha
  v226+2b -m*c   v230+b .. v236+b scratch
  s40 c = scale*log2(e)   s41 -inf   s42 8.0   s[44:45] K source of tile t+2   s[46:47] V source of
  tile t+1   s48 / s49 bytes per K / V tile   s50 LDS address of this wave's part of buffer 0
  s51 trips left   s[52:53], s[60:61] scratch   s[54:55], s[58:59] rows whose reference moved in the
  tile before (zero on entry)   s56 scratch
"""
import os
import re

# experiment switches (comma separated in LVX_GEN_OPTS); none is set in a normal build
OPTS = dict((o.split("=") + ["1"])[:2] for o in os.environ.get("LVX_GEN_OPTS", "").split(",") if o)
MFMA = "v_mfma_f32_32x32x16_bf16"

NB = 2
SC = [[0, 32], [64, 96]]            # score sets [block][set]
PB = [128, 144]
STG, KA, VA, DO = 160, 200, 208, 216
MI, LI, AL = [220, 221], [222, 223], [224, 225]
NMC = [226, 228]
MX, T0, T1, RS1 = [230, 231], [232, 233], [234, 235], [236, 237]
AACC, AQ = [0, 64], [128, 160]
RMASK = ["s[54:55]", "s[58:59]"]
CMASK = ["s[52:53]", "s[60:61]"]
NSLOT, AHEAD, WBATCH = 10, int(OPTS.get("ahead", 8)), int(OPTS.get("wbatch", 2))
TILE = 16384


def vr(base, n=1):
    return f"v{base}" if n == 1 else f"v[{base}:{base + n - 1}]"


def ar(base, n=1):
    return f"a{base}" if n == 1 else f"a[{base}:{base + n - 1}]"


class Stream:
    """Instruction list with a model of the in-order LDS return queue for s_waitcnt lgkmcnt."""

    def __init__(self):
        self.out = []
        self.lds_issued = 0
        self.ready_after = {}   # operand id -> number of LDS reads issued when its last read was issued

    def emit(self, s):
        if isinstance(s, list):     # instructions that must stay together
            for x in s:
                self.emit(x)
            return
        if "nodma" in OPTS and (s.startswith("global_load_lds") or s.startswith("s_add_i32 m0")):
            return
        if "novalu" in OPTS and s.startswith("v_") and not s.startswith("v_mfma") and not s.startswith("v_acc"):
            return
        self.out.append(s)

    def lds_read(self, text, op):
        if "nolds" not in OPTS:
            self.out.append(text)
        self.lds_issued += 1
        self.ready_after[op] = self.lds_issued

    def wait_op(self, op):
        n = self.lds_issued - self.ready_after[op]
        self.out.append(f"s_waitcnt lgkmcnt({min(n, 15)})")


def exp_group(b, cur, j, nmc, first):
    """P^T k-step j of block b from its score set cur: registers 8j..8j+7 of s0 (j < 2) or s1.
    Exponentials and their consumers are kept at least two instructions apart."""
    base = SC[b][cur] + (16 if j >= 2 else 0) + 8 * (j & 1)
    ins = []
    pend = []
    for e in range(4):
        r0, r1 = base + 2 * e, base + 2 * e + 1
        ins.append(f"v_fma_f32 v{r0}, v{r0}, s40, v{nmc}")
        ins.append(f"v_fma_f32 v{r1}, v{r1}, s40, v{nmc}")
        ins.append(f"v_exp_f32 v{r0}, v{r0}")
        ins.append(f"v_exp_f32 v{r1}, v{r1}")
        ins += pend
        pend = []
        if first and e == 0:
            pend.append(f"v_add_f32 v{RS1[b]}, v{r0}, v{r1}")
        else:
            pend.append(f"v_add_f32 v{LI[b]}, v{LI[b]}, v{r0}")
            pend.append(f"v_add_f32 v{RS1[b]}, v{RS1[b]}, v{r1}")
        pend.append(f"v_cvt_pk_bf16_f32 v{PB[b] + 4 * j + e}, v{r0}, v{r1}")
    ins.append("s_nop 0")
    ins += pend
    return ins


SLOW = []       # out-of-line code: the reference moves of the tiles of the loop
N_SLOW = [0]


def next_max(b, nxt):
    """Row maximum of the next tile's scores of block b and the test whether any row's reference
    maximum has to move (its maximum grew by more than 2^8 since the reference was set, or there was
    none).  The move itself - alpha, the new reference and -m*c - is rare and sits behind the loop."""
    s0, s1 = SC[b][nxt], SC[b][nxt] + 16
    mx, t0, t1, mi, al, nmc = MX[b], T0[b], T1[b], MI[b], AL[b], NMC[b]
    ins = [f"v_max3_f32 v{mx}, v{s0}, v{s1}, v{s0 + 1}"]
    for v in range(2, 16):
        ins.append(f"v_max3_f32 v{mx}, v{mx}, v{s1 + v - 1}, v{s0 + v}")
    ins.append(f"v_max_f32 v{mx}, v{mx}, v{s1 + 15}")
    n = N_SLOW[0]
    N_SLOW[0] += 1
    ins += [
        f"v_mov_b32 v{t0}, v{mx}",
        "s_nop 1",
        f"v_permlane32_swap_b32 v{mx}, v{t0}",
        "s_nop 1",
        f"v_max3_f32 v{mx}, v{mx}, v{t0}, v{mi}",
        # candidate reference mx*c against the current m*c: move when the difference exceeds 8 (or is not
        # a number: no reference yet) and mx is finite
        f"v_mul_f32 v{t0}, s40, v{mx}",
        f"v_fma_f32 v{t0}, -s40, v{mi}, v{t0}",
        f"v_cmp_neq_f32 vcc, s41, v{mx}",
        f"v_cmp_nge_f32 {CMASK[b]}, s42, v{t0}",
        [f"s_and_b64 {RMASK[b]}, vcc, {CMASK[b]}",
         f"s_cbranch_scc1 LVX_FWDW_MOVE{n}_%=",
         f"LVX_FWDW_MOVED{n}_%=:"],
    ]
    SLOW.extend([
        f"LVX_FWDW_MOVE{n}_%=:",
        f"v_mul_f32 v{t0}, s40, v{mx}",
        f"v_fma_f32 v{t1}, s40, v{mi}, -v{t0}",
        f"v_exp_f32 v{t1}, v{t1}",
        "s_nop 1",
        f"v_cndmask_b32 v{al}, 1.0, v{t1}, {RMASK[b]}",
        f"v_cndmask_b32 v{mi}, v{mi}, v{mx}, {RMASK[b]}",
        "s_nop 0",
        f"v_mul_f32 v{nmc}, v{mi}, -s40",
        f"v_cmp_neq_f32 vcc, s41, v{mi}",
        "s_nop 1",
        f"v_cndmask_b32 v{nmc}, 0, v{nmc}, vcc",
        f"s_branch LVX_FWDW_MOVED{n}_%=",
    ])
    return ins


def rescale(b, tag, e):
    """O^T and l of block b times alpha, for the rare tile in which some row's reference maximum moved
    (behind the loop, like the move itself).  The accumulators are out of reach of the VALU: sixteen at
    a time travel through the operand slots, which hold nothing at the top of a tile."""
    e([f"s_cmp_lg_u64 {RMASK[b]}, 0", f"s_cbranch_scc1 LVX_FWDW_RESC{tag}{b}_%=", f"LVX_FWDW_RESCD{tag}{b}_%=:"])
    out = [f"LVX_FWDW_RESC{tag}{b}_%=:", "s_nop 15", "s_nop 3", f"v_mul_f32 v{LI[b]}, v{LI[b]}, v{AL[b]}"]
    for c in range(4):
        for r in range(16):
            out.append(f"v_accvgpr_read_b32 v{STG + r}, a{AACC[b] + 16 * c + r}")
        for r in range(16):
            out.append(f"v_mul_f32 v{STG + r}, v{AL[b]}, v{STG + r}")
        for r in range(16):
            out.append(f"v_accvgpr_write_b32 a{AACC[b] + 16 * c + r}, v{STG + r}")
    out += ["s_nop 3", f"s_branch LVX_FWDW_RESCD{tag}{b}_%="]
    SLOW.extend(out)


def tile(par, do_cur=True, do_next=True, do_dma=True, top=True):
    """One key tile t of the pipelined loop (par = t & 1 relative to the first tile of the run).
    do_cur : P(t) from the current scores, O += V(t)^T P(t)
    do_next: S(t+1) = K(t+1) Q^T into the other score set, its row maximum and reference move
    do_dma : request K(t+2) and V(t+1)"""
    cur, nxt = par, par ^ 1
    st = Stream()
    e = st.emit
    tag = f"{par}{int(do_cur)}{int(do_next)}"
    if top:
        # K(t+1) and V(t) have landed; nobody reads K(t) / V(t-1) any more
        e("s_waitcnt vmcnt(0)")
        e("s_barrier")
    if do_cur:
        for b in range(NB):
            rescale(b, tag, e)

    # operand n: 0..15 = K (k-step n/2, key half n%2) from buffer par^1; 16..31 = V (k-step j = (n-16)/4,
    # d tile (n-16)%4) from buffer par
    ops = (list(range(16)) if do_next else []) + (list(range(16, 32)) if do_cur else [])

    def read_op(n):
        slot = STG + 4 * (n % NSLOT)
        if n < 16:
            kk, half = n // 2, n % 2
            st.lds_read(f"ds_read_b128 {vr(slot, 4)}, v{KA + kk} offset:{(par ^ 1) * 2 * TILE + half * 8192}", n)
        else:
            j, dt = (n - 16) // 4, (n - 16) % 4
            off = par * 2 * TILE + j * 4096
            st.lds_read(f"ds_read_b64_tr_b16 {vr(slot, 2)}, v{VA + 2 * dt} offset:{off}", n)
            st.lds_read(f"ds_read_b64_tr_b16 {vr(slot + 2, 2)}, v{VA + 2 * dt + 1} offset:{off}", n)

    for n in ops[:AHEAD]:
        read_op(n)

    # VALU work of the tile in dependency order; group_end[(b, j)] = how many of them must have been
    # emitted before the MFMAs that read P^T k-step j of block b
    valu, group_end, first_max = [], {}, 10 ** 9
    n_pre = 0
    if do_cur:
        for j in range(4):
            for b in range(NB):
                valu += exp_group(b, cur, j, NMC[b], j == 0)
                group_end[(b, j)] = len(valu)
            if j == 0:
                n_pre = len(valu)       # one group per block before the first MFMA covers the K read latency
            if j == 1 and not do_next:
                n_pre = len(valu)       # without an S phase the first two P operands have to be there anyway
        for b in range(NB):
            valu.append(f"v_add_f32 v{LI[b]}, v{LI[b]}, v{RS1[b]}")
    if do_next:
        first_max = len(valu)
        for b in range(NB):
            valu += next_max(b, nxt)
    for s in valu[:n_pre]:
        e(s)
    pos = n_pre
    # global -> LDS loads: K(t+2) into K buffer par, V(t+1) into V buffer par^1
    dma = []
    if do_dma:
        for j in range(4):
            dma.append((f"s_add_i32 m0, s50, {par * 2 * TILE + j * 4096}", f"global_load_lds_dwordx4 v{DO + j}, s[44:45]"))
        for j in range(4):
            dma.append((f"s_add_i32 m0, s50, {(par ^ 1) * 2 * TILE + TILE + j * 4096}", f"global_load_lds_dwordx4 v{DO + j}, s[46:47]"))
    s1, s2 = int(OPTS.get("s1", 4)), int(OPTS.get("s2", 5))
    n_mfma = 0
    last_s = -100       # index of the last S MFMA
    for i, k in enumerate(ops):
        if i % WBATCH == 0:         # one wait covers the operands of the next few MFMA pairs
            st.wait_op(ops[min(i + WBATCH - 1, len(ops) - 1)])
        slot = STG + 4 * (k % NSLOT)
        for b in range(NB):
            if k < 16:
                kk, half = k // 2, k % 2
                d = SC[b][nxt] + 16 * half
                c = "0" if kk == 0 else vr(d, 16)
                e(f"{MFMA} {vr(d, 16)}, {vr(slot, 4)}, {ar(AQ[b] + 4 * kk, 4)}, {c}")
                last_s = n_mfma
            else:
                j, dt = (k - 16) // 4, (k - 16) % 4
                assert pos >= group_end[(b, j)], f"P^T k-step {j} of block {b} is not ready at operand {k}"
                a = AACC[b] + 16 * dt
                e(f"{MFMA} {ar(a, 16)}, {vr(slot, 4)}, {vr(PB[b] + 4 * j, 4)}, {ar(a, 16)}")
            n_mfma += 1
            if b == NB - 1:
                if i + AHEAD < len(ops):
                    read_op(ops[i + AHEAD])
                if dma and k < 16 and k % 2 == 1:
                    x, y = dma[k // 2]
                    e(x)
                    e(y)
                if do_dma and k == 15:
                    # the run has 2 * trips + 1 tiles: the last even tile must not move the K source past the
                    # last tile (the odd tile after it then requests that tile once more, which nobody reads)
                    if par == 0:
                        e("s_cmp_lg_u32 s51, 1")
                        e("s_cselect_b32 s56, s48, 0")
                        e("s_add_u32 s44, s44, s56")
                    else:
                        e("s_add_u32 s44, s44, s48")
                    e("s_addc_u32 s45, s45, 0")
                    e("s_add_u32 s46, s46, s49")
                    e("s_addc_u32 s47, s47, 0")
            take = (s1 if k < 16 else s2) if do_next else 7
            if i == len(ops) - 1 and b == NB - 1:
                take = len(valu) - pos
            for _ in range(take):
                if pos >= len(valu):
                    break
                # the row maximum reads the scores the S MFMAs wrote: not before the last of them has had
                # its wait states - with the V MFMAs behind it, no earlier than three MFMAs later
                if pos >= first_max and (n_mfma - 1 < last_s + 4 or k < 16):
                    break
                e(valu[pos])
                pos += 1
    if pos < len(valu):     # S phase alone (prologue): the maximum follows the last MFMA
        e("s_nop 15")
        e("s_nop 3")
        for s in valu[pos:]:
            e(s)
    return st.out


def check(ins):
    """Hazard lint of one tile's stream (conservative): distance in instructions, an s_nop N counting N+1."""
    def regs(tok):
        tok = tok.strip().lstrip("-")
        m = re.match(r"([va])\[(\d+):(\d+)\]$", tok)
        if m:
            return set((m.group(1), r) for r in range(int(m.group(2)), int(m.group(3)) + 1))
        m = re.match(r"([va])(\d+)$", tok)
        return {(m.group(1), int(m.group(2)))} if m else set()
    hist = []   # (kind, written regs, weight)
    for line in ins:
        if line.endswith(":"):
            continue
        op, _, rest = line.partition(" ")
        toks = [t for t in rest.split(",")] if rest else []
        toks = [t.split(" offset")[0] for t in toks]
        weight = 1
        if op == "s_nop":
            weight = int(rest) + 1
        wr, rd = set(), set()
        kind = "other"
        if op.startswith("v_mfma"):
            kind = "mfma"
            wr = regs(toks[0])
            rd = regs(toks[1]) | regs(toks[2]) | regs(toks[3])
        elif op.startswith("v_cmp"):
            kind = "valu"
            rd = set().union(*[regs(t) for t in toks[1:]])
        elif op.startswith("v_permlane"):
            kind = "valu"
            wr = regs(toks[0]) | regs(toks[1])
            rd = wr
        elif op.startswith("v_"):
            kind = "trans" if op.startswith("v_exp") else "valu"
            wr = regs(toks[0])
            rd = set().union(*[regs(t) for t in toks[1:]]) if len(toks) > 1 else set()
        elif op.startswith("ds_read"):
            kind = "lds"
            wr = regs(toks[0])
            rd = regs(toks[1])
        elif op.startswith("global_load_lds"):
            kind = "vmem"
            rd = regs(toks[0])
        dist = 0
        for pk, pw, pwt in reversed(hist):
            if pk == "mfma" and kind != "mfma" and (pw & (rd | wr)) and dist < 14:
                raise SystemExit(f"hazard: {line} touches an MFMA result after {dist} wait states")
            if pk in ("valu", "trans") and kind == "mfma" and (pw & rd) and dist < 3:
                raise SystemExit(f"hazard: {line} reads a VALU result after {dist} wait states")
            if pk == "trans" and kind in ("valu", "trans") and (pw & rd) and dist < 2:
                raise SystemExit(f"hazard: {line} reads a transcendental result after {dist} wait states")
            if pk == "valu" and op.startswith("v_permlane") and (pw & rd) and dist < 2:
                raise SystemExit(f"hazard: {line} reads a VALU result after {dist} wait states")
            dist += pwt
            if dist > 40:
                break
        hist.append((kind, wr, weight))


def main():
    # Entry: O^T and Q^T move up into the accumulation registers.
    pro = []
    for b in range(NB):
        for r in range(64):
            pro.append(f"v_accvgpr_write_b32 a{AACC[b] + r}, v{64 * b + r}")
        for r in range(32):
            pro.append(f"v_accvgpr_write_b32 a{AQ[b] + r}, v{128 + 32 * b + r}")
    # All loads of the run are the loop's own.  s[44:45] / s[46:47] point at K / V of its first tile.
    pro += ["s_barrier"]
    for j in range(4):
        pro += [f"s_add_i32 m0, s50, {j * 4096}", f"global_load_lds_dwordx4 v{DO + j}, s[44:45]"]
    for j in range(4):
        pro += [f"s_add_i32 m0, s50, {TILE + j * 4096}", f"global_load_lds_dwordx4 v{DO + j}, s[46:47]"]
    pro += ["s_add_u32 s44, s44, s48", "s_addc_u32 s45, s45, 0", "s_add_u32 s46, s46, s49", "s_addc_u32 s47, s47, 0"]
    for j in range(4):
        pro += [f"s_add_i32 m0, s50, {2 * TILE + j * 4096}", f"global_load_lds_dwordx4 v{DO + j}, s[44:45]"]
    pro += ["s_add_u32 s44, s44, s48", "s_addc_u32 s45, s45, 0"]
    pro += ["s_waitcnt vmcnt(4)", "s_barrier"]
    for b in range(NB):     # -m*c of the reference the block arrives with (0 without one)
        pro += [f"v_mul_f32 v{NMC[b]}, v{MI[b]}, -s40", f"v_cmp_neq_f32 vcc, s41, v{MI[b]}", "s_nop 1",
                f"v_cndmask_b32 v{NMC[b]}, 0, v{NMC[b]}, vcc"]
    # scores of the first tile (from K buffer 0 into score set A: the S phase of an odd tile)
    pro += tile(1, do_cur=False, do_next=True, do_dma=False, top=False)
    t0, t1 = tile(0), tile(1)
    fin = tile(0, do_cur=True, do_next=False, do_dma=False)
    check(pro + t0 + t1 + t0 + t1 + fin)
    lines = pro + ["LVX_FWDW_LOOP_%=:"] + t0 + t1
    lines += ["s_sub_i32 s51, s51, 1", "s_cmp_lg_u32 s51, 0", "s_cbranch_scc1 LVX_FWDW_LOOP_%="]
    lines += fin + ["s_nop 15", "s_nop 3"]
    lines += ["s_branch LVX_FWDW_END_%="] + SLOW + ["LVX_FWDW_END_%=:"]
    # Exit: O^T and Q^T come back down.
    for b in range(NB):
        for r in range(64):
            lines.append(f"v_accvgpr_read_b32 v{64 * b + r}, a{AACC[b] + r}")
        for r in range(32):
            lines.append(f"v_accvgpr_read_b32 v{128 + 32 * b + r}, a{AQ[b] + r}")
    lines += ["s_nop 3"]
    print("// generated by gen_fwd_loop_wide.py - do not edit")
    for l in lines:
        print(f'"{l}\\n"')


main()
