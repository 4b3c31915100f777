"""Writes the hand-scheduled steady-state loops of the gfx950 backward kernel (lvx_bwd.hip):

    python gen_bwd_loop.py p > lvx_bwd_loop_p.inc      (P-waves: S, P = exp2(..), dV^T)
    python gen_bwd_loop.py d > lvx_bwd_loop_d.inc      (D-waves: dP, dS, dK^T)

Each is one inline-asm statement with every register named here.  One trip does six steps (the
six tile buffers of each ring and the two-deep P / dS^T buffers then sit at immediate offsets);
the first step of a trip is a step i with i % 6 == 3.  Inside a step the 16 MFMAs of a wave are
spread over its other instructions (LDS operand reads eight operands ahead, the exponentials or
the dS arithmetic of an earlier tile, the global -> LDS loads and the dS^T copy-out), so that a
wave keeps the matrix pipe fed by itself.

LDS map in bytes (lvx_bwd.hip): Q ring 6 x 8192 at 0, dO ring at 49152, dS^T tiles 2 x 10240 at
98304, P hand-over 2 x 8192 at 118784; the metadata records 6 x 512 bytes are a separate array.

Registers, both roles: v[0:63] resident accumulators (dV^T / dK^T)   v[64:95] resident B operands
(K rows / V rows)   v[96:111], v[112:127] the two score sets (raw S / dP), swapping every step
v[128:159] eight operand slots  v[200:207] row-read addresses into "its" ring (P: Q, D: dO)
v[208:215] transposing-read addresses into the other ring.   s40 scale*log2(e) (P) / scale (D)
P-waves: v[168:175] P packed   v[176:191] LSE*log2(e) of 16 rows   v[192:199] dS^T copy-out data
  v216 P hand-over write address   v217 metadata read address   v218 dS^T copy-out read address
  v219, v220 copy-out global offsets   v221..v224 global offsets of the four tile loads   v225 of
  the metadata load
  s41 / s42 bytes per Q / dO tile   s[44:45] Q, s[46:47] dO, s[48:49] metadata, s[50:51] dS^T
  workspace address of the next tile to request   s52 tiles left in its head   s53 tiles per head
  s[54:55] / s[56:57] / s[60:61] what a head change adds to the Q / dO / workspace address
  s62 LDS address of this wave's part of Q buffer 0   s63 of the metadata records   s64 trips
  s65 1 in wave 0 (it requests the metadata)   s[66:77] workspace addresses of the tiles in flight
  s[78:79] scratch
D-waves: v[168:175] P handed over   v[176:183] dS packed   v[184:199] delta*scale of 16 rows
  v216 P hand-over read address   v217 metadata read address   v218 dS^T staging write address
"""
import os
import re
import sys

# experiment switches (comma separated in LVX_GEN_OPTS); none is set in a normal build
OPTS = dict((o.split("=") + ["1"])[:2] for o in os.environ.get("LVX_GEN_OPTS", "").split(",") if o)
ROLE = sys.argv[1] if len(sys.argv) > 1 else "p"
for _o in list(OPTS):      # a switch for one role only: p_novalu, d_nolds, ...
    if _o.startswith(ROLE + "_"):
        OPTS[_o[2:]] = OPTS[_o]
F16 = False
MFMA = "v_mfma_f32_32x32x16_bf16"

ACC, BREG, SET, STG, RA, TA = 0, 64, (96, 112), 128, 200, 208
NSLOT, AHEAD = 8, 7
TILE_B, DO_RING, DST_B, DST_SZ, PB_SZ, META_SZ = 8192, 49152, 98304, 10240, 8192, 512
# P role
PU, LSE, CPD = 168, 176, 192
A_PB, A_META, A_CP, G_CP0, G_CP1, G_DMA, G_META = 216, 217, 218, 219, 220, 221, 225
# D role
DSU, DELTA, TMP = 176, 184, 219


def vr(base, n=1):
    return f"v{base}" if n == 1 else f"v[{base}:{base + n - 1}]"


def sr(base, n=1):
    return f"s{base}" if n == 1 else f"s[{base}:{base + n - 1}]"


class Stream:
    """Instruction list with a model of the in-order LDS queue for s_waitcnt lgkmcnt."""

    def __init__(self, seed=None):
        self.out = []
        self.n_lds = 0
        self.tag = {}
        self.done = 0           # LDS operations 1 .. done are known to have completed
        self.last_write = 0     # position of the last ds_write
        if seed is not None:    # what the step before left in flight: see carry_over()
            self.n_lds = seed["n"]
            self.tag = dict(seed["tag"])

    def emit(self, s):
        if "nodma" in OPTS and (s.startswith("global_load_lds") or s.startswith("s_add_i32 m0")):
            return
        if "nostore" in OPTS and s.startswith("global_store"):
            return
        if "novalu" in OPTS and s.startswith("v_") and not s.startswith("v_mfma"):
            return
        if "nomfma" in OPTS and s.startswith("v_mfma"):
            return
        if "nobar" in OPTS and s.startswith("s_barrier"):
            return
        self.out.append(s)

    def lds(self, text, tag=None):
        if "nolds" in OPTS and "_tr_" in text or "nolds" in OPTS and text.startswith("ds_read_b128 v[1") and int(text.split("[")[1].split(":")[0]) < 160:
            text = None
        if text is not None:
            self.out.append(text)
        self.n_lds += 1
        if tag is not None:
            self.tag[tag] = self.n_lds
        if text is not None and text.startswith("ds_write"):
            self.last_write = self.n_lds

    def wait(self, tag):
        if self.tag[tag] <= self.done:      # an earlier wait of this step covers it
            return
        n = min(self.n_lds - self.tag[tag], 15)
        self.out.append(f"s_waitcnt lgkmcnt({n})")
        self.done = self.n_lds - n

    def carry_over(self, u_next):
        """What a step leaves to the next one: the LDS operations it issued after its last write (the
        next step waits at its top until only these are in flight: LDS operations complete in order, so
        the writes other waves are about to read have then landed) and, among them, the reads of the
        first operands of the next step."""
        n = self.n_lds - self.last_write
        tag = {t: pos - self.last_write for t, pos in self.tag.items()     # <= 0: read before the write
               if isinstance(t, tuple) and t[0] == "op" and t[1] == u_next}
        assert len(tag) == AHEAD and n <= 15, (n, tag)
        return {"n": n, "tag": tag}

    def wait_needed(self, tag):
        return self.n_lds - self.tag[tag]


def spread(st, mfmas, side, shares):
    """Emit MFMA k (a callable writing its wait + instruction), then shares[k] entries of side."""
    pos = 0
    for k, m in enumerate(mfmas):
        m()
        take = shares[k] if k + 1 < len(mfmas) else 10 ** 6
        while take > 0 and pos < len(side):
            x = side[pos]
            pos += 1
            if isinstance(x, list):     # a branch and what it jumps over stay together
                for y in x:
                    st.emit(y)
                take -= len(x)
            else:
                x() if callable(x) else st.emit(x)
                take -= 1
    assert pos == len(side), (pos, len(side))


def p_read_op(st, u, n):
    """LDS read of operand n of P-wave step u: 0..7 Q rows of tile i (k-step n), 8..15 dO^T of tile i-1."""
    sl_i, sl_p = (u + 3) % 6, (u + 2) % 6
    slot = STG + 4 * (n % NSLOT)
    if n < 8:
        st.lds(f"ds_read_b128 {vr(slot, 4)}, v{RA + n} offset:{sl_i * TILE_B}", ("op", u, n))
    else:
        j, dt = (n - 8) // 4, (n - 8) % 4
        off = sl_p * TILE_B + j * 4096
        st.lds(f"ds_read_b64_tr_b16 {vr(slot, 2)}, v{TA + 2 * dt} offset:{off}")
        st.lds(f"ds_read_b64_tr_b16 {vr(slot + 2, 2)}, v{TA + 2 * dt + 1} offset:{off}", ("op", u, n))


def p_fetch(u, ahead):
    """Request of tile i + ahead by a P-wave in step u, and the walk to the tile after it."""
    sl_f = (u + 3 + ahead) % 6
    ws_new = 66 + 2 * sl_f
    f = [["s_cmp_eq_u32 s65, 0", f"s_cbranch_scc1 LVX_BWD_NOMETA{u}{ahead}_%=", f"s_add_i32 m0, s63, {sl_f * META_SZ}",
          f"global_load_lds_dword v{G_META}, s[48:49]", f"LVX_BWD_NOMETA{u}{ahead}_%=:"]]
    for n, (base, src) in enumerate(((0, "s[44:45]"), (1024, "s[44:45]"), (DO_RING, "s[46:47]"), (DO_RING + 1024, "s[46:47]"))):
        f.append(f"s_add_i32 m0, s62, {sl_f * TILE_B + base}")
        f.append(f"global_load_lds_dwordx4 v{G_DMA + n}, {src}")
    f.append(f"s_mov_b64 {sr(ws_new, 2)}, s[50:51]")
    f += ["s_add_u32 s44, s44, s41", "s_addc_u32 s45, s45, 0", "s_add_u32 s46, s46, s42", "s_addc_u32 s47, s47, 0",
          "s_add_u32 s48, s48, 256", "s_addc_u32 s49, s49, 0", "s_add_u32 s50, s50, 8192", "s_addc_u32 s51, s51, 0",
          ["s_sub_i32 s52, s52, 1", "s_cmp_lg_u32 s52, 0", f"s_cbranch_scc1 LVX_BWD_SAMEHEAD{u}{ahead}_%=",
           "s_add_u32 s44, s44, s54", "s_addc_u32 s45, s45, s55", "s_add_u32 s46, s46, s56", "s_addc_u32 s47, s47, s57",
           "s_add_u32 s50, s50, s60", "s_addc_u32 s51, s51, s61", "s_mov_b32 s52, s53", f"LVX_BWD_SAMEHEAD{u}{ahead}_%=:"]]
    return f


def flat(items):
    out = []
    for x in items:
        out += x if isinstance(x, list) else [x]
    return out


def p_step(u, seed):
    """P-wave step i, i % 6 == (u + 3) % 6.  Operands 0..6 were read in the step before."""
    st = Stream(seed)
    e = st.emit
    sl_p = (u + 2) % 6
    par = u & 1                                                  # (i + 1) & 1: P(i-1) hand-over, dS^T(i-3)
    carry, new = SET[u & 1], SET[(u + 1) & 1]
    # tile i+1 has landed: after its loads this wave issued 2 stores, 4 (wave 0: 5) loads and 2 stores
    e("s_waitcnt vmcnt(6)" if "storefirst" in OPTS else "s_waitcnt vmcnt(8)")
    e(f"s_waitcnt lgkmcnt({st.n_lds})")
    e("s_barrier")
    for vg in range(4):
        st.lds(f"ds_read_b128 {vr(LSE + 4 * vg, 4)}, v{A_META} offset:{sl_p * META_SZ + vg * 32}", ("lse", vg))

    # P(i-1) = exp2(S(i-1) * c - LSE), packed
    valu = []
    for vg in range(4):
        valu.append(lambda vg=vg: st.wait(("lse", vg)))
        for r in range(4):
            v = 4 * vg + r
            valu.append(f"v_fma_f32 v{carry + v}, v{carry + v}, s40, -v{LSE + v}")
        for r in range(4):
            valu.append(f"v_exp_f32 v{carry + 4 * vg + r}, v{carry + 4 * vg + r}")
        if vg >= 1:
            for e2 in range(2):
                v = 4 * (vg - 1) + 2 * e2
                valu.append(f"v_cvt_pk_bf16_f32 v{PU + v // 2}, v{carry + v}, v{carry + v + 1}")
    valu.append("s_nop 0")
    for e2 in range(2):
        v = 12 + 2 * e2
        valu.append(f"v_cvt_pk_bf16_f32 v{PU + v // 2}, v{carry + v}, v{carry + v + 1}")
    # hand P over to the D-wave
    valu.append(lambda: st.lds(f"ds_write_b128 v{A_PB}, {vr(PU, 4)} offset:{par * PB_SZ}"))
    valu.append(lambda: st.lds(f"ds_write_b128 v{A_PB}, {vr(PU + 4, 4)} offset:{par * PB_SZ + 1024}"))

    # second half: request of tile i+3 and the walk, dS^T(i-3) copy-out.  The loads go first: the wait
    # at the top of a step then leaves the two stores of the step before last in flight as well
    tail = []
    tail.append(lambda: st.lds(f"ds_read_b128 {vr(CPD, 4)}, v{A_CP} offset:{par * DST_SZ}", "cp0"))
    tail.append(lambda: st.lds(f"ds_read_b128 {vr(CPD + 4, 4)}, v{A_CP} offset:{par * DST_SZ + 5120}", "cp1"))
    ws_old = 66 + 2 * (u % 6)          # workspace address of tile i-3 (tile i+3 takes its place below)
    fetch = p_fetch(u, 3)
    if u == 5:      # the last step of the last trip requests nothing: the steps after the loop do
        fetch = [["s_cmp_eq_u32 s64, 1", "s_cbranch_scc1 LVX_BWD_NOFETCH_%="] + flat(fetch) + ["LVX_BWD_NOFETCH_%=:"]]
    store = [lambda: st.wait("cp0"), f"global_store_dwordx4 v{G_CP0}, {vr(CPD, 4)}, {sr(ws_old, 2)}",
             lambda: st.wait("cp1"), f"global_store_dwordx4 v{G_CP1}, {vr(CPD + 4, 4)}, {sr(ws_old, 2)}"]
    if "storefirst" in OPTS:
        tail += store + fetch
    else:
        # the stores read the workspace address of tile i-3 before the walk overwrites it: keep a copy
        tail += [f"s_mov_b64 s[78:79], {sr(ws_old, 2)}"] + fetch
        store[1] = f"global_store_dwordx4 v{G_CP0}, {vr(CPD, 4)}, s[78:79]"
        store[3] = f"global_store_dwordx4 v{G_CP1}, {vr(CPD + 4, 4)}, s[78:79]"
        tail += store

    mf = []
    for k in range(16):
        def m(k=k):
            st.wait(("op", u, k))
            slot = STG + 4 * (k % NSLOT)
            if k < 8:
                c = "0" if k == 0 else vr(new, 16)
                e(f"{MFMA} {vr(new, 16)}, {vr(slot, 4)}, {vr(BREG + 4 * k, 4)}, {c}")
            else:
                j, dt = (k - 8) // 4, (k - 8) % 4
                e(f"{MFMA} {vr(ACC + 16 * dt, 16)}, {vr(slot, 4)}, {vr(PU + 4 * j, 4)}, {vr(ACC + 16 * dt, 16)}")
            if k + AHEAD < 16:
                p_read_op(st, u, k + AHEAD)
            else:
                p_read_op(st, (u + 1) % 6, k + AHEAD - 16)
        mf.append(m)
    side = valu + tail
    nv = len(valu)
    nt = sum(len(x) if isinstance(x, list) else 1 for x in tail)
    shares = [(nv + 7) // 8] * 8 + [(nt + 6) // 7] * 8
    spread(st, mf, side, shares)
    return st.out, st.carry_over((u + 1) % 6)


def p_prologue():
    """Before the first trip: the operands the first step expects to have been read, and tile i+2."""
    st = Stream()
    st.emit("s_waitcnt vmcnt(0)")
    st.emit("s_waitcnt lgkmcnt(0)")
    st.emit("s_barrier")
    for n in range(AHEAD):
        p_read_op(st, 0, n)
    for y in flat(p_fetch(0, 2)):
        st.emit(y)
    st.emit("s_waitcnt lgkmcnt(0)")     # the first step counts on no more in flight than a step leaves
    return st.out


def d_read_op(st, u, n):
    """LDS read of operand n of D-wave step u: 0..7 dO rows of tile i-1, 8..15 Q^T of tile i-2."""
    sl_p, sl_pp = (u + 2) % 6, (u + 1) % 6
    slot = STG + 4 * (n % NSLOT)
    if n < 8:
        st.lds(f"ds_read_b128 {vr(slot, 4)}, v{RA + n} offset:{sl_p * TILE_B}", ("op", u, n))
    else:
        j, dt = (n - 8) // 4, (n - 8) % 4
        off = sl_pp * TILE_B + j * 4096
        st.lds(f"ds_read_b64_tr_b16 {vr(slot, 2)}, v{TA + 2 * dt} offset:{off}")
        st.lds(f"ds_read_b64_tr_b16 {vr(slot + 2, 2)}, v{TA + 2 * dt + 1} offset:{off}", ("op", u, n))


def d_step(u, seed):
    """D-wave step i, i % 6 == (u + 3) % 6.  Operands 0..6 were read in the step before."""
    st = Stream(seed)
    e = st.emit
    sl_pp = (u + 1) % 6                        # buffer of tile i-2 (Q^T, metadata)
    par = (u + 1) & 1                          # i & 1: P(i-2) hand-over, dS^T(i-2) staging
    carry, new = SET[u & 1], SET[(u + 1) & 1]
    e(f"s_waitcnt lgkmcnt({st.n_lds})")
    e("s_barrier")
    st.lds(f"ds_read_b128 {vr(PU, 4)}, v{A_PB} offset:{par * PB_SZ}", ("pu", 0))
    st.lds(f"ds_read_b128 {vr(PU + 4, 4)}, v{A_PB} offset:{par * PB_SZ + 1024}", ("pu", 1))
    for q in range(4):
        st.lds(f"ds_read_b128 {vr(DELTA + 4 * q, 4)}, v{A_META} offset:{sl_pp * META_SZ + 128 + q * 32}", ("dl", q))

    # scale * dS(i-2) = P(i-2) * (dP(i-2) * scale - delta * scale), packed
    valu = []
    t = [TMP, TMP + 1, TMP + 2, TMP + 3]
    for q in range(4):          # registers 4q .. 4q+3 of the dP set; P pairs PU[2q], PU[2q+1]
        valu.append(lambda q=q: st.wait(("dl", q)))      # the P reads were issued before the delta reads
        for r in range(4):
            v = 4 * q + r
            valu.append(f"v_fma_f32 v{carry + v}, v{carry + v}, s40, -v{DELTA + v}")
        valu.append(f"v_lshlrev_b32 v{t[0]}, 16, v{PU + 2 * q}")
        valu.append(f"v_and_b32 v{t[1]}, 0xffff0000, v{PU + 2 * q}")
        valu.append(f"v_lshlrev_b32 v{t[2]}, 16, v{PU + 2 * q + 1}")
        valu.append(f"v_and_b32 v{t[3]}, 0xffff0000, v{PU + 2 * q + 1}")
        for r in range(4):
            v = 4 * q + r
            valu.append(f"v_mul_f32 v{carry + v}, v{t[r]}, v{carry + v}")
        valu.append(f"v_cvt_pk_bf16_f32 v{DSU + 2 * q}, v{carry + 4 * q}, v{carry + 4 * q + 1}")
        valu.append(f"v_cvt_pk_bf16_f32 v{DSU + 2 * q + 1}, v{carry + 4 * q + 2}, v{carry + 4 * q + 3}")
    for vg in range(4):
        valu.append(lambda vg=vg: st.lds(f"ds_write_b64 v{218}, {vr(DSU + 2 * vg, 2)} offset:{par * DST_SZ + 16 * vg}"))

    mf = []
    for k in range(16):
        def m(k=k):
            st.wait(("op", u, k))
            slot = STG + 4 * (k % NSLOT)
            if k < 8:
                c = "0" if k == 0 else vr(new, 16)
                e(f"{MFMA} {vr(new, 16)}, {vr(slot, 4)}, {vr(BREG + 4 * k, 4)}, {c}")
            else:
                j, dt = (k - 8) // 4, (k - 8) % 4
                e(f"{MFMA} {vr(ACC + 16 * dt, 16)}, {vr(slot, 4)}, {vr(DSU + 4 * j, 4)}, {vr(ACC + 16 * dt, 16)}")
            if k + AHEAD < 16:
                d_read_op(st, u, k + AHEAD)
            else:
                d_read_op(st, (u + 1) % 6, k + AHEAD - 16)
        mf.append(m)
    shares = [6] * 8 + [4, 4, 4, 2, 2, 2, 0, 0]
    spread(st, mf, valu, shares)
    return st.out, st.carry_over((u + 1) % 6)


def d_prologue():
    st = Stream()
    st.emit("s_waitcnt lgkmcnt(0)")
    st.emit("s_barrier")
    for n in range(AHEAD):
        d_read_op(st, 0, n)
    st.emit("s_waitcnt lgkmcnt(0)")     # the first step counts on no more in flight than a step leaves
    return st.out


def check(ins):
    """Hazard lint (conservative): distance in issue slots, an s_nop N counting N + 1."""
    def regs(tok):
        tok = tok.strip().lstrip("-")
        m = re.match(r"v\[(\d+):(\d+)\]$", tok)
        if m:
            return set(range(int(m.group(1)), int(m.group(2)) + 1))
        m = re.match(r"v(\d+)$", tok)
        return {int(m.group(1))} if m else set()
    hist = []
    for line in ins:
        if line.endswith(":"):
            continue
        op, _, rest = line.partition(" ")
        toks = [t.split(" offset")[0] for t in rest.split(",")] if rest else []
        weight = int(rest) + 1 if op == "s_nop" else 1
        wr, rd, kind = set(), set(), "other"
        if op.startswith("v_mfma"):
            kind, wr = "mfma", regs(toks[0])
            rd = regs(toks[1]) | regs(toks[2]) | regs(toks[3])
        elif op.startswith("v_"):
            kind = "trans" if op.startswith("v_exp") else "valu"
            wr = regs(toks[0])
            rd = set().union(*[regs(x) for x in toks[1:]]) if len(toks) > 1 else set()
        elif op.startswith("ds_read"):
            kind, wr, rd = "lds", regs(toks[0]), regs(toks[1])
        elif op.startswith("ds_write"):
            kind, rd = "lds", regs(toks[0]) | regs(toks[1])
        elif op.startswith("global_store"):
            kind, rd = "vmem", regs(toks[0]) | regs(toks[1])
        elif op.startswith("global_load_lds"):
            kind, rd = "vmem", regs(toks[0])
        dist = 0
        for pk, pw, pwt in reversed(hist):
            if pk == "mfma" and kind != "mfma" and (pw & (rd | wr)) and dist < 14:
                raise SystemExit(f"hazard: {line} touches an MFMA result after {dist} slots")
            if pk in ("valu", "trans") and kind == "mfma" and (pw & rd) and dist < 3:
                raise SystemExit(f"hazard: {line} reads a VALU result after {dist} slots")
            if pk == "trans" and kind in ("valu", "trans") and (pw & rd) and dist < 2:
                raise SystemExit(f"hazard: {line} reads a transcendental result after {dist} slots")
            dist += pwt
            if dist > 40:
                break
        hist.append((kind, wr, weight))


def main():
    step = p_step if ROLE == "p" else d_step
    # what step 5 leaves to step 0 of the next trip: every step issues the same LDS operations in the
    # same order, so a dry run of one step tells
    _, seed = step(5, {"n": AHEAD, "tag": {("op", 5, k): k + 1 for k in range(AHEAD)}})
    body = []
    for u in range(6):
        ins, left = step(u, seed)
        assert u == 5 or left == {"n": seed["n"], "tag": {("op", u + 1, t[2]): p for t, p in seed["tag"].items()}}, (left, seed)
        seed = left
        body += [x for x in ins if x is not None]
    check(body + body)
    cnt = "s64"
    lines = (p_prologue() if ROLE == "p" else d_prologue()) + ["LVX_BWD_LOOP_%=:"] + body + [f"s_sub_i32 {cnt}, {cnt}, 1", f"s_cmp_lg_u32 {cnt}, 0", "s_cbranch_scc1 LVX_BWD_LOOP_%=",
                                           "s_waitcnt lgkmcnt(0)", "s_nop 15", "s_nop 3"]
    print("// generated by gen_bwd_loop.py - do not edit")
    for l in lines:
        print(f'"{l}\\n"')


main()
