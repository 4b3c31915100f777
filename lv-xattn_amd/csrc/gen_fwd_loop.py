"""Writes lvx_fwd_loop.inc: the hand-scheduled steady-state loop of the gfx950 forward kernel.

    python gen_fwd_loop.py [bf16|f16] > lvx_fwd_loop_bf16.inc

The loop is one inline-asm statement of lvx_fwd.hip with every register named here.  One trip
does two key tiles (the two LDS buffers and the two score sets swap roles, so all LDS offsets
are immediates).  Per tile t the matrix pipe gets 32 MFMAs back to back in program order -
S(t+1) = K(t+1) Q^T, then O += V(t)^T P(t) - and between any two of them sit a few of the other
instructions of the tile: the exponentials of tile t, the row maximum of tile t+1, the LDS
operand reads ten operands ahead, the global -> LDS loads of K(t+2) and V(t+1).  A wave whose
MFMAs are spaced like this keeps the pipe busy by itself; a wave that issues its MFMAs as one
block and its VALU work as another does not (measured: the two blocks take the sum of their
times, also across the two waves that share a SIMD).

Register map (must match the constraints of the asm statement in lvx_fwd.hip):
  v[0:63]    O^T accumulators, four 32x32 tiles        v[64:95]   Q^T, eight B operands
  v[96:127]  scores, set A   v[128:159] scores, set B  v[160:175] P^T, four B operands
  v[176:215] ten operand slots (LDS read targets)      v[224:231] K read addresses (per k-step)
  v[232:239] V read addresses (d tile x half)          v[240:243] global offsets of the 4 row groups
  v244 m  v245 l  v246 alpha  v247/v248 -m*c of the current / next tile (swapping)  v249.. scratch
  s40 c = scale*log2(e)   s41 -inf   s42 8.0   s[44:45] K source of tile t+2   s[46:47] V source of
  tile t+1   s48 / s49 bytes per K / V tile   s50 LDS address of this wave's part of buffer 0
  s51 trips left   s[52:53], s[54:55] scratch
"""
import os
import sys

# experiment switches (comma separated in LVX_GEN_OPTS); none is set in a normal build
OPTS = dict((o.split("=") + ["1"])[:2] for o in os.environ.get("LVX_GEN_OPTS", "").split(",") if o)
F16 = len(sys.argv) > 1 and sys.argv[1] == "f16"
MFMA = "v_mfma_f32_32x32x16_f16" if F16 else "v_mfma_f32_32x32x16_bf16"

ACC, Q, SA, SB, P, STG, KA, VA, DO = 0, 64, 96, 128, 160, 176, 224, 232, 240
MI, LI, AL, NMC, MX, T0, T1, RS1, T2 = 244, 245, 246, (247, 248), 249, 250, 251, 252, 253
NSLOT, AHEAD = 10, int(OPTS.get("ahead", 8))
TILE = 16384


def vr(base, n=1):
    return f"v{base}" if n == 1 else f"v[{base}:{base + n - 1}]"


class Stream:
    """Instruction list with a model of the in-order LDS return queue for s_waitcnt lgkmcnt."""

    def __init__(self):
        self.out = []
        self.lds_issued = 0
        self.ready_after = {}   # operand id -> number of LDS reads issued when its last read was issued

    def emit(self, s):
        if "nodma" in OPTS and (s.startswith("global_load_lds") or s.startswith("s_add_i32 m0")):
            return
        if "halfdma" in OPTS and (s.startswith("global_load_lds") or s.startswith("s_add_i32 m0")):
            self.ndma = getattr(self, "ndma", 0) + 1
            if (self.ndma - 1) // 2 % 2:
                return
        if "novalu" in OPTS and s.startswith("v_") and not s.startswith("v_mfma") and not s.startswith("v_mul_f32 v2"):
            return
        self.out.append(s)

    def lds_read(self, text, op):
        if "nolds" not in OPTS and not ("halflds" in OPTS and (op & 1)):
            self.out.append(text)
        self.lds_issued += 1
        self.ready_after[op] = self.lds_issued

    def wait_op(self, op):
        n = self.lds_issued - self.ready_after[op]
        self.out.append(f"s_waitcnt lgkmcnt({min(n, 15)})")


def exp_group(cur, j, nmc, first):
    """P^T k-step j from scores cur: registers 8j..8j+7 of s0 (j < 2) or s1.  Returns instructions;
    exponentials and their consumers are kept at least two instructions apart."""
    base = cur + (16 if j >= 2 else 0) + 8 * (j & 1)
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
            pend.append(f"v_add_f32 v{RS1}, v{r0}, v{r1}")
        else:
            pend.append(f"v_add_f32 v{LI}, v{LI}, v{r0}")
            pend.append(f"v_add_f32 v{RS1}, v{RS1}, v{r1}")
        if F16:
            pend.append(f"v_cvt_f16_f32 v{r0}, v{r0}")
            pend.append(f"v_cvt_f16_f32 v{r1}, v{r1}")
            pend.append(f"v_pack_b32_f16 v{P + 4 * j + e}, v{r0}, v{r1}")
        else:
            pend.append(f"v_cvt_pk_bf16_f32 v{P + 4 * j + e}, v{r0}, v{r1}")
    ins.append("s_nop 0")
    ins += pend
    return ins


def next_max(nxt, nmc_next):
    """Row maximum of the next tile's scores, then the lazy move of the reference maximum."""
    s0, s1 = nxt, nxt + 16
    ins = [f"v_max3_f32 v{MX}, v{s0}, v{s1}, v{s0 + 1}"]
    for v in range(2, 16):
        ins.append(f"v_max3_f32 v{MX}, v{MX}, v{s1 + v - 1}, v{s0 + v}")
    ins.append(f"v_max_f32 v{MX}, v{MX}, v{s1 + 15}")
    ins += [
        f"v_mov_b32 v{T0}, v{MX}",
        "s_nop 1",
        f"v_permlane32_swap_b32 v{MX}, v{T0}",
        "s_nop 1",
        f"v_max3_f32 v{MX}, v{MX}, v{T0}, v{MI}",
        # candidate reference mcand = mx*c, current m*c; move when mcand - m*c > 8 and mx is finite
        f"v_mul_f32 v{T0}, s40, v{MX}",
        f"v_fma_f32 v{T1}, s40, v{MI}, -v{T0}",
        f"v_exp_f32 v{T1}, v{T1}",
        f"v_fma_f32 v{T0}, -s40, v{MI}, v{T0}",
        f"v_cmp_neq_f32 vcc, s41, v{MX}",
        f"v_cmp_nge_f32 s[52:53], s42, v{T0}",
        "s_and_b64 s[52:53], vcc, s[52:53]",
        "s_nop 1",
        f"v_cndmask_b32 v{AL}, 1.0, v{T1}, s[52:53]",
        f"v_cndmask_b32 v{MI}, v{MI}, v{MX}, s[52:53]",
        "s_nop 0",
        f"v_cmp_neq_f32 vcc, 1.0, v{AL}",
        "s_mov_b64 s[54:55], vcc",
        f"v_mul_f32 v{nmc_next}, v{MI}, -s40",
        f"v_cmp_neq_f32 vcc, s41, v{MI}",
        "s_nop 1",
        f"v_cndmask_b32 v{nmc_next}, 0, v{nmc_next}, vcc",
    ]
    return ins


def tile(par, do_cur=True, do_next=True, do_dma=True, top=True):
    """One key tile t of the pipelined loop (par = t & 1 relative to the first tile of the run).
    do_cur : P(t) from the current scores, O += V(t)^T P(t)
    do_next: S(t+1) = K(t+1) Q^T into the other score set, its row maximum and reference move
    do_dma : request K(t+2) and V(t+1)"""
    cur, nxt = (SA, SB) if par == 0 else (SB, SA)
    nmc, nmc_next = NMC[par], NMC[par ^ 1]
    st = Stream()
    e = st.emit
    tag = f"{par}{int(do_cur)}{int(do_next)}"
    if top:
        # K(t+1) and V(t) have landed; nobody reads K(t) / V(t-1) any more
        e("s_waitcnt vmcnt(0)")
        e("s_barrier")
    if do_cur:
        e("s_cmp_eq_u64 s[54:55], 0")
        e(f"s_cbranch_scc1 LVX_FWD_NORESC{tag}_%=")
        e("s_nop 15")
        for r in range(64):
            e(f"v_mul_f32 v{ACC + r}, v{AL}, v{ACC + r}")
        e(f"LVX_FWD_NORESC{tag}_%=:")

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

    # VALU work of the tile, in dependency order
    valu, n_pre, first_max = [], 0, 10 ** 9
    if do_cur:
        valu.append(f"v_mul_f32 v{LI}, v{LI}, v{AL}")
        for j in range(4):
            valu += exp_group(cur, j, nmc, j == 0)
        valu.append(f"v_add_f32 v{LI}, v{LI}, v{RS1}")
        # exponentials that run before the first MFMA: one group covers the latency of the K reads;
        # without an S phase the first two P operands have to be there anyway
        n_pre = 1 + len(exp_group(cur, 0, nmc, True)) * (1 if do_next else 2)
    if do_next:
        first_max = len(valu)
        valu += next_max(nxt, nmc_next)
    for s in valu[:n_pre]:
        e(s)
    rest = valu[n_pre:]
    first_max -= n_pre
    # global -> LDS loads: K(t+2) into K buffer par, V(t+1) into V buffer par^1; one after every other MFMA
    dma = []
    if do_dma:
        for j in range(4):
            dma.append((f"s_add_i32 m0, s50, {par * 2 * TILE + j * 4096}", f"global_load_lds_dwordx4 v{DO + j}, s[44:45]"))
        for j in range(4):
            dma.append((f"s_add_i32 m0, s50, {(par ^ 1) * 2 * TILE + TILE + j * 4096}", f"global_load_lds_dwordx4 v{DO + j}, s[46:47]"))
    # VALU instructions per MFMA slot: lighter while the loads are being issued
    share = {k: int(OPTS.get("s1", 3)) if k < 16 else int(OPTS.get("s2", 5)) for k in range(32)}
    if not do_next:
        share = {k: 7 for k in range(32)}
    pos = 0
    last_s = -100     # position (in MFMAs) of the last S MFMA
    for i, k in enumerate(ops):
        st.wait_op(k)
        slot = STG + 4 * (k % NSLOT)
        if k < 16:
            kk, half = k // 2, k % 2
            d = nxt + 16 * half
            c = "0" if kk == 0 else vr(d, 16)
            e(f"{MFMA} {vr(d, 16)}, {vr(slot, 4)}, {vr(Q + 4 * kk, 4)}, {c}")
            last_s = i
        else:
            j, dt = (k - 16) // 4, (k - 16) % 4
            e(f"{MFMA} {vr(ACC + 16 * dt, 16)}, {vr(slot, 4)}, {vr(P + 4 * j, 4)}, {vr(ACC + 16 * dt, 16)}")
        if i + AHEAD < len(ops):
            read_op(ops[i + AHEAD])
        if dma and k < 16 and k % 2 == 1:
            a, b = dma[k // 2]
            e(a)
            e(b)
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
        take = share[k]
        if i == len(ops) - 1:
            take = len(rest) - pos
        for _ in range(take):
            if pos >= len(rest):
                break
            # the row maximum reads the scores the S MFMAs wrote: not before the last of them has had
            # its wait states - with the V MFMAs behind it, no earlier than three MFMAs later
            if pos >= first_max and (i < last_s + 3 or (k < 16)):
                break
            e(rest[pos])
            pos += 1
    if pos < len(rest):     # S phase alone (prologue): the maximum follows the last MFMA
        e("s_nop 15")
        for s in rest[pos:]:
            e(s)
    return st.out


def check(ins):
    """Hazard lint of one tile's stream (conservative): distance in instructions, an s_nop N counting N+1."""
    import re
    def regs(tok):
        tok = tok.strip().lstrip("-")
        m = re.match(r"v\[(\d+):(\d+)\]$", tok)
        if m:
            return set(range(int(m.group(1)), int(m.group(2)) + 1))
        m = re.match(r"v(\d+)$", tok)
        return {int(m.group(1))} if m else set()
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
    # Entry: all loads of the run are the loop's own.  s[44:45] / s[46:47] point at K / V of its first tile.
    pro = ["s_barrier"]
    for j in range(4):
        pro += [f"s_add_i32 m0, s50, {j * 4096}", f"global_load_lds_dwordx4 v{DO + j}, s[44:45]"]
    for j in range(4):
        pro += [f"s_add_i32 m0, s50, {TILE + j * 4096}", f"global_load_lds_dwordx4 v{DO + j}, s[46:47]"]
    pro += ["s_add_u32 s44, s44, s48", "s_addc_u32 s45, s45, 0", "s_add_u32 s46, s46, s49", "s_addc_u32 s47, s47, 0"]
    for j in range(4):
        pro += [f"s_add_i32 m0, s50, {2 * TILE + j * 4096}", f"global_load_lds_dwordx4 v{DO + j}, s[44:45]"]
    pro += ["s_add_u32 s44, s44, s48", "s_addc_u32 s45, s45, 0"]
    pro += ["s_waitcnt vmcnt(4)", "s_barrier"]
    # scores of the first tile (from K buffer 0 into score set A: the S phase of an odd tile)
    pro += tile(1, do_cur=False, do_next=True, do_dma=False, top=False)
    t0, t1 = tile(0), tile(1)
    fin = tile(0, do_cur=True, do_next=False, do_dma=False)
    check(pro + t0 + t1 + t0 + t1 + fin)
    lines = pro + ["LVX_FWD_LOOP_%=:"] + t0 + t1
    lines += ["s_sub_i32 s51, s51, 1", "s_cmp_lg_u32 s51, 0", "s_cbranch_scc1 LVX_FWD_LOOP_%="]
    lines += fin + ["s_nop 15", "s_nop 3"]
    print("// generated by gen_fwd_loop.py - do not edit")
    for l in lines:
        print(f'"{l}\\n"')


main()
