// Cross-attention backward for gfx950 from the saved LSE and delta:
//   P = exp(scale*Q K^T - LSE);  dV = P^T dO;  dP = dO V^T;
//   dS = P * (dP - delta);  dK = scale * dS^T Q;  dQ = scale * dS K.
//
// Mapping.  A work-group owns a block of 128 visual tokens of one kv head and
// streams every text row of the window for every q head of the GQA group past
// it, 32 rows at a time.  It has 8 waves, two per SIMD, in two roles; waves w
// and w+4 share token slice 32w..32w+31 of the block:
//   P-wave  (w)   : S = Q K^T, P = exp2(..), dV^T += dO^T P     K rows + dV^T resident
//   D-wave  (w+4) : dP = dO V^T, dS = P (dP - delta) scale,
//                   dK^T += Q^T dS                              V rows + dK^T resident
// so each wave keeps 64 accumulator registers and 32 operand registers for the
// whole kernel (the sum over the q heads of the group and over all rows never
// leaves the register file) and fits two to a SIMD: while one wave waits for
// LDS or runs its exp2/multiplies, the other feeds the MFMA pipe.  P travels
// from the P-wave to the D-wave as bf16 through LDS (32 bytes per lane), one
// step behind, so the one barrier per step also orders that hand-over.
//
// dQ = scale * dS K sums over ALL tokens, i.e. over every work-group of the kv
// head.  Adding 51 partial tiles per row with fp32 atomics costs more than the
// whole rest of the kernel on this machine (atomic adds sustain about 1.3 TB/s),
// so dQ is not formed here: the D-waves gather scale*dS (bf16) in LDS and the
// group streams it to a workspace in HBM, one contiguous 8 KB tile
// [128 tokens][32 rows] per step, indexed [b, h, token block, row tile]; a
// batched GEMM (launched by the caller right after) contracts it with K.  The workspace costs 2 bytes per (row, token, head),
// written once and read once.
//
// All MFMA are 32x32x16 bf16.  A operands come from LDS.  The Q and dO tiles
// ([32 rows][128] bf16, 8 KiB each) go from global memory straight into LDS
// with global_load_lds_dwordx4, two steps ahead, into rings of six buffers;
// the load writes 64 lanes x 16 bytes contiguously, so rows are not padded:
// the 16-byte chunk c of row r is kept at position c ^ f(r),
// f(r) = ((r & 3) << 2) | ((r >> 2) & 3), which makes both access patterns
// conflict-free on ONE copy of a tile - Q / dO rows by 16-byte reads, Q^T /
// dO^T by the transposing LDS read, the latter addressed in the accumulator's
// row order so that P / dS go from the registers straight into the next MFMA
// as B operands.  Every wave requests all LDS operands of a step before its
// first MFMA, so their latency is paid once per step.
#include <type_traits>

#include "lvx_common.hpp"
#include "lvx_kernels.hpp"

namespace lvx {

namespace {

constexpr int D = 128;
constexpr int BN = 128;       // visual tokens per work-group
constexpr int BM = 32;        // text rows per step
constexpr int NT = 512;       // threads per work-group
constexpr int DSS = BM + 8;   // row stride of the dS^T tile [token][row]

// LDS map (uint16 units): a ring of six Q tiles, a ring of six dO tiles (each ring within the 64 KiB an LDS
// instruction's immediate offset reaches from one address register), unpadded; two dS^T tiles; two P
// hand-over buffers
constexpr int TILE_ELEMS = BM * D;             // one Q or dO tile (8 KiB)
constexpr int NQD = 6;
constexpr int DST_ELEMS = BN * DSS;
constexpr int PB_ELEMS = 4 * 2 * 64 * 8;       // P hand-over: [slice][half][lane][16 bytes] as uint16
constexpr int OFF_Q = 0;                       // x NQD
constexpr int OFF_DO = OFF_Q + NQD * TILE_ELEMS; // x NQD
constexpr int OFF_DST = OFF_DO + NQD * TILE_ELEMS; // x2
constexpr int OFF_PB = OFF_DST + 2 * DST_ELEMS;  // x2
constexpr int LOOP_ELEMS = OFF_PB + 2 * PB_ELEMS;
constexpr int EPS = D + 1;                          // row stride (floats) of the epilogue's transposed tile
constexpr int EPI_ELEMS = 8 * 32 * EPS * 2;         // 8 waves x [32 tokens][128 + 1] floats, in uint16 units
constexpr int SMEM_ELEMS = LOOP_ELEMS > EPI_ELEMS ? LOOP_ELEMS : EPI_ELEMS;

constexpr float LOG2E = 1.4426950408889634f;

// registers the hand-scheduled loops use besides their operands (see gen_bwd_loop.py)
#define LVX_BWD_LOOP_CLOBBERS "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120", "v121", "v122", "v123", "v124", "v125", "v126", "v127", "v128", "v129", "v130", "v131", "v132", "v133", "v134", "v135", "v136", "v137", "v138", "v139", "v140", "v141", "v142", "v143", "v144", "v145", "v146", "v147", "v148", "v149", "v150", "v151", "v152", "v153", "v154", "v155", "v156", "v157", "v158", "v159", "v160", "v161", "v162", "v163", "v164", "v165", "v166", "v167", "v168", "v169", "v170", "v171", "v172", "v173", "v174", "v175", "v176", "v177", "v178", "v179", "v180", "v181", "v182", "v183", "v184", "v185", "v186", "v187", "v188", "v189", "v190", "v191", "v192", "v193", "v194", "v195", "v196", "v197", "v198", "v199"

// BIAS: a dense fp32 bias joins the exponent, P = exp2(S*c + bias*log2e - LSE*log2e).
// DH: head dimension, 16, 32, 64 or 128.  The LDS tiles keep their 256-byte rows and chunk
// permutation whatever DH is: below 128 only the first DH / 8 chunks of a row hold data (the
// lanes that would load the others repeat a chunk of the same row), and the k-steps of S / dP
// and the 32-wide blocks of dV^T / dK^T past DH do not exist.  With 16 the one block of dV^T /
// dK^T is half real: its upper 16 rows are products with those repeated chunks, never stored.
template <int DH, bool MASKED, bool BIAS, bool F16>
__global__ __launch_bounds__(NT, 1) void bwd_kernel(const BwdParams p) {
    using E = Elt<F16>;
    static_assert(DH == 16 || DH == 32 || DH == 64 || DH == 128, "head dimension");
    constexpr int NKK = DH / 16, NDT = DH >= 32 ? DH / 32 : 1;
    __shared__ __attribute__((aligned(1024))) uint16_t smem[SMEM_ELEMS];
    // per-row metadata of a staged tile, one per tile buffer: 8 x 16 bytes each of
    // LSE*log2e, delta*scale, kv_start, kv_end
    __shared__ __attribute__((aligned(256))) u32x4 meta_s4[NQD][BM];

    // Work-group ids are dealt to the 8 XCDs round-robin.  XCD x takes the token blocks
    // [x * blocks_per_xcd, (x + 1) * blocks_per_xcd) of the list (b, kv head, block), so that the
    // work-groups of a kv head share an L2: first `whole_blocks` of them with one work-group
    // each, then `mid_blocks` with q_splits work-groups each, then the others with q_splits2
    // each - the longer work-groups first.  (A placement hint only: every (block, range) is
    // produced exactly once whatever the hardware does with the ids.)
    const int xcd = blockIdx.x % 8, local = blockIdx.x / 8;
    const int blk0 = xcd * p.blocks_per_xcd;
    const int nblk = min(p.blocks_per_xcd, p.n_blocks - blk0);
    const int whole = max(0, min(p.whole_blocks, nblk));
    const int mid = max(0, min(p.mid_blocks, nblk - whole));
    int blk, sp = 0, S = 1;
    if (local < whole) {
        blk = blk0 + local;
    } else if (local < whole + mid * p.q_splits) {
        const int l2 = local - whole;
        S = p.q_splits;
        sp = l2 % S;
        blk = blk0 + whole + l2 / S;
    } else {
        const int l3 = local - whole - mid * p.q_splits;
        S = p.q_splits2;
        sp = l3 % S;
        blk = blk0 + whole + mid + l3 / S;
        if (blk >= blk0 + nblk) return;
    }
    const int kblk = blk % p.n_kv_blocks;
    const int bh = blk / p.n_kv_blocks;
    const int b = bh % p.B;            // samples interleaved: ragged samples then share the tail of the launch
    const int hk = bh / p.B;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int slice = wave & 3;
    const bool d_role = wave >= 4;

    int kv_len = p.Lkv;
    if (p.kv_len) kv_len = min(p.kv_len[b], p.Lkv);
    const int kvb = kblk * BN;
    const int my_kv = kvb + 32 * slice + l32;
    const bool kv_valid = my_kv < kv_len;
    const int slice_lo = kvb + 32 * slice;              // this wave's 32 tokens
    const bool slice_valid = slice_lo + 32 <= kv_len;   // all of them inside the sample
    const bool tail_block = kvb + BN > kv_len;

    // steps of this work-group: a contiguous range of the (head, row tile) list
    const int n_qtiles = (p.row_end - p.row_begin + BM - 1) / BM;
    // with an interval mask only the listed runs of tiles are visited (kept in scalar
    // registers), and the splits share that shorter walk evenly
    int run_s[4] = {0, 0, 0, 0}, run_n[4] = {n_qtiles, 0, 0, 0};
    int n_live = n_qtiles;
    if (MASKED && p.live_runs) {
        const int32_t* lr = p.live_runs + ((int64_t)b * p.n_kv_blocks + kblk) * 8;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            run_s[i] = __builtin_amdgcn_readfirstlane(lr[2 * i]);
            run_n[i] = __builtin_amdgcn_readfirstlane(lr[2 * i + 1]);
        }
        n_live = run_n[0] + run_n[1] + run_n[2] + run_n[3];
    }
    const int split_steps = (p.G * n_live + S - 1) / S;
    auto sel4 = [](int r, const int (&a)[4]) { return r == 0 ? a[0] : r == 1 ? a[1] : r == 2 ? a[2] : a[3]; };
    const int it_lo = sp * split_steps;
    const int n_iter = (kvb < kv_len) ? max(0, min(split_steps, p.G * n_live - it_lo)) : 0;
    // nothing to visit and nothing to overwrite: done (bf16 outputs, mode 0, still get their zeros)
    // a block that its work-group owns alone is written by it directly, also when others are shared
    const bool alone = p.dkv_mode == 2 && S == 1;
    const int dkv_mode = alone ? p.whole_mode : p.dkv_mode;
    if (n_iter == 0 && dkv_mode != 0) return;

    // ---- resident B operand: this wave's K rows (P-wave) or V rows (D-wave)
    bf16x8 breg[8];     // [NKK .. 8) stay unused when DH < 128
    {
        const uint16_t* base = d_role ? p.v + b * p.vs.b + hk * p.vs.h + (int64_t)my_kv * p.vs.s
                                      : p.k + b * p.ks.b + hk * p.ks.h + (int64_t)my_kv * p.ks.s;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) breg[kk] = as_bf16x8(ldg16(base + (kk < NKK ? kk : 0) * 16 + g * 8, kv_valid));
    }
    // ---- resident accumulator: dV^T (P-wave) or dK^T (D-wave), [128 d][32 tokens]
    f32x16 acc[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[dt][v] = 0.f;

    const float c = p.scale_log2e;

    // global -> LDS is the P-waves' job (their step is the shorter one): P-wave w moves
    // rows 8w..8w+7 of the Q tile and of the dO tile as two 1 KiB loads each (4 rows
    // per load); lane i fills position i & 15 of row 4 ch + (i >> 4), ch = 2w, 2w+1.
    const int ld_r = 8 * slice + (lane >> 4);          // first of the two rows, the other is 4 further
    const uint32_t ld_c0 = (uint32_t)(((lane & 15) ^ (((lane >> 4) << 2) | ((2 * slice) & 3))) & (DH / 8 - 1)) * 16u;
    const uint32_t ld_c1 = (uint32_t)(((lane & 15) ^ (((lane >> 4) << 2) | ((2 * slice + 1) & 3))) & (DH / 8 - 1)) * 16u;
    const uint32_t qrow_b = (uint32_t)p.qs.s * 2u, dorow_b = (uint32_t)p.dos.s * 2u;   // bytes per text row
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const uint32_t meta0 = (uint32_t)(uintptr_t)&meta_s4[0][0];
    // per-lane offsets: transposing operand reads (rows in accumulator order),
    // P hand-over slot, dS^T copy-out (512 chunks of 16 bytes, one per thread)
    // rows: 16 bytes at row * 256 + ((2 kk + g) ^ f(row)) * 16
    const uint32_t row_rd = (uint32_t)(l32 * 256);
    const uint32_t row_h = (uint32_t)((g ^ (((l32 & 3) << 2) | ((l32 >> 2) & 3))) << 4);
    // transposed, rows in accumulator order: first half rows 16 j + 4 g + r, second
    // half 8 rows further down (its f differs in bit 1); add j * 4096
    uint32_t t_rd[4][2];
    {
        const int r = (lane & 15) >> 2, t = lane & 3, u = (lane >> 4) & 1;
        const int low = (2 * u + (t >> 1)) ^ g;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
            t_rd[dt][0] = (uint32_t)((4 * g + r) * 256 + (4 * (dt ^ r) + low) * 16 + (t & 1) * 8);
            t_rd[dt][1] = (uint32_t)((4 * g + r + 8) * 256 + (4 * (dt ^ r) + (low ^ 2)) * 16 + (t & 1) * 8);
        }
    }
    const int pb_off = slice * (2 * 64 * 8) + lane * 8;
    // dS^T copy-out, also by the P-waves: 512 chunks of 16 bytes, two per thread (tokens t >> 2 and 64 + (t >> 2))
    const int cp_token = (tid & 255) >> 2, cp_part = tid & 3;
    // workspace tile (b, h, token block, row tile): [128 tokens][32 rows], 8 KB, contiguous
    uint16_t* ws_lane = p.ds_ws + (int64_t)kblk * p.ws_ld + cp_token * BM + cp_part * 8;

    // The walk over (head of the group, 32-row tile): per-head base addresses are
    // re-derived only when the head changes, everything else advances by constants.
    int cur_gi = 0, cur_run = 0, cur_qt = 0, cur_left = 1;    // cur_left: tiles left in the run, this one included
    if (n_iter > 0) {
        cur_gi = it_lo / n_live;
        int idx = it_lo % n_live;
        while (idx >= sel4(cur_run, run_n)) { idx -= sel4(cur_run, run_n); ++cur_run; }
        cur_qt = sel4(cur_run, run_s) + idx;
        cur_left = sel4(cur_run, run_n) - idx;
    }
    const char* q_head = nullptr;      // Q, dO of (b, head)
    const char* do_head = nullptr;
    const float* meta_head = nullptr;  // metadata records of (b, head)
    int64_t ws_head = 0;               // dS^T workspace offset of (b, head), elements
    auto enter_head = [&]() {
        const int h = hk * p.G + cur_gi;
        q_head = reinterpret_cast<const char*>(p.q + b * p.qs.b + h * p.qs.h);
        do_head = reinterpret_cast<const char*>(p.dout + b * p.dos.b + h * p.dos.h);
        meta_head = p.meta + ((int64_t)b * p.Hq + h) * n_qtiles * 64;
        ws_head = ((int64_t)b * p.Hq + h) * p.ws_bh;
    };
    enter_head();

    // Every load is unconditional and goes straight to LDS: rows past the window are
    // clamped to its last row (their LSE record is +inf, so P = 0 and nothing they
    // carry reaches a result).  Wave 0 also fetches the tile's metadata record
    // (32 x LSE*log2e, 32 x delta*scale; 256 bytes) and, with a mask, the rows'
    // key intervals, ahead of its tile loads so that "tile landed" implies both.
    auto prefetch = [&](int buf) {
        const int r0 = p.row_begin + cur_qt * BM;
        if (wave == 0) {
            const uint32_t mslot = meta0 + (uint32_t)buf * (BM * 16);
            dma4(reinterpret_cast<const char*>(meta_head + cur_qt * 64), (uint32_t)lane * 4u, mslot);
            if (MASKED) {
                const int32_t* iv = (lane < 32 ? p.kv_start : p.kv_end) + (int64_t)b * p.Lq + min(r0 + l32, p.row_end - 1);
                dma4_addr(reinterpret_cast<const char*>(iv), mslot + 256);
            }
        }
        const uint32_t row0 = (uint32_t)min(r0 + ld_r, p.row_end - 1);
        const uint32_t row1 = (uint32_t)min(r0 + ld_r + 4, p.row_end - 1);
        const uint32_t slot = lds0 + (uint32_t)buf * (TILE_ELEMS * 2) + (uint32_t)slice * 2048u;
        dma16(q_head, row0 * qrow_b + ld_c0, slot);
        dma16(q_head, row1 * qrow_b + ld_c1, slot + 1024);
        dma16(do_head, row0 * dorow_b + ld_c0, slot + OFF_DO * 2);
        dma16(do_head, row1 * dorow_b + ld_c1, slot + OFF_DO * 2 + 1024);
    };
    auto advance = [&]() {   // next (head, row tile) of the walk, wrapping
        ++cur_qt;
        if (--cur_left > 0) return;
        if (++cur_run == 4 || sel4(cur_run, run_n) == 0) {
            cur_run = 0;
            if (++cur_gi == p.G) cur_gi = 0;
            enter_head();
        }
        cur_qt = sel4(cur_run, run_s);
        cur_left = sel4(cur_run, run_n);
    };

    // the finished dS^T tile goes to HBM as one contiguous 8 KB block
    auto copy_out = [&](const uint16_t* dst, int64_t ws_off) {
        const u32x4 a = *reinterpret_cast<const u32x4*>(dst + cp_token * DSS + cp_part * 8);
        const u32x4 c2 = *reinterpret_cast<const u32x4*>(dst + (cp_token + 64) * DSS + cp_part * 8);
        *reinterpret_cast<u32x4*>(ws_lane + ws_off) = a;
        *reinterpret_cast<u32x4*>(ws_lane + ws_off + 64 * BM) = c2;
    };

    // The work on a tile is spread over three steps so that, inside every wave, the
    // MFMAs of one tile and the VALU work of an earlier tile are independent and
    // overlap (on top of the overlap between the two waves of a SIMD):
    //   step i, P-wave: S(i) = Q K_w^T                     || P(i-1) = exp2(S(i-1)*c - LSE*log2e), masked
    //                   then hand P(i-1) over, dV_w^T += dO(i-1)^T P(i-1)
    //   step i, D-wave: dP(i-1) = dO V_w^T                 || dS(i-2) = P(i-2) (dP(i-2)*scale - delta*scale)
    //                   then dS^T(i-2) to LDS, dK_w^T += Q(i-2)^T dS(i-2)
    //   step i, all   : request tile i+2, copy dS^T(i-3) out
    // Flags say which halves exist at the edges of the walk; they are compile-time
    // constants in the steady-state loop.
    auto p_step = [&](auto tail_c, bool s_live, bool pv_live, const uint16_t* tile_cur, const uint16_t* tile_prev,
                      const u32x4* meta, uint16_t* pbuf, f32x16& s_carry, int64_t bias_off, int bias_r0)
                      __attribute__((always_inline)) {
        constexpr bool TAIL = decltype(tail_c)::value;
        float bv[16];
        if (BIAS && pv_live) {   // bias of (row 8 vg + 4 g + r of the previous tile, this lane's token)
            const float* bp = p.bias + bias_off + min(my_kv, p.Lkv - 1);
            const int last = p.row_end - 1 - bias_r0;
#pragma unroll
            for (int v = 0; v < 16; ++v) bv[v] = bp[(int64_t)min(8 * (v >> 2) + 4 * g + (v & 3), last) * p.bias_r];
        }
        const char* qt = reinterpret_cast<const char*>(tile_cur);     // Q of tile i
        const char* dot = reinterpret_cast<const char*>(tile_prev);   // dO of tile i-1
        bf16x8 qa[8];
        u32x2 da[4][2][2];
        // MASKED: lane l looks at the key interval of row l of the previous tile (requested
        // first, so the answer is there long before it is needed)
        int iv_s = 0, iv_e = 0;
        if (MASKED && pv_live) {
            const int32_t* iv = reinterpret_cast<const int32_t*>(meta + 16);
            iv_s = iv[l32];
            iv_e = iv[32 + l32];
        }
        if (s_live) {
#pragma unroll
            for (int kk = 0; kk < NKK; ++kk)
                qa[kk] = *reinterpret_cast<const bf16x8*>(qt + row_rd + ((uint32_t)(kk * 32) ^ row_h));
        }
        __builtin_amdgcn_sched_barrier(0);
        f32x16 s_new;
        if (s_live) {
#pragma unroll
            for (int v = 0; v < 16; ++v) s_new[v] = 0.f;
#pragma unroll
            for (int kk = 0; kk < NKK; ++kk) s_new = E::mfma(qa[kk], breg[kk], s_new);
        }
        if (pv_live) {
            // dO^T operands: requested once the S operands are consumed; they land while
            // the exp2 phase runs in the shadow of the S MFMAs
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    da[dt][j][0] = lds_read_tr16(reinterpret_cast<const uint16_t*>(dot + t_rd[dt][0] + j * 4096));
                    da[dt][j][1] = lds_read_tr16(reinterpret_cast<const uint16_t*>(dot + t_rd[dt][1] + j * 4096));
                }
            f32x16 s = s_carry;
#pragma unroll
            for (int vg = 0; vg < 4; ++vg) {
                const f32x4 l4 = __builtin_bit_cast(f32x4, meta[2 * vg + g]);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float off = BIAS ? fmaf(bv[4 * vg + r], LOG2E, -l4[r]) : -l4[r];
                    s[4 * vg + r] = __builtin_amdgcn_exp2f(fmaf(s[4 * vg + r], c, off));
                }
            }
            if (MASKED) {
                // most (tile, token slice) pairs a mask leaves alive are alive as a whole; only a
                // slice that some row of the tile cuts is masked element by element
                const bool cut = iv_s > slice_lo || iv_e < slice_lo + 32;
                if (!slice_valid || __builtin_amdgcn_ballot_w64(cut) != 0) {
#pragma unroll
                    for (int vg = 0; vg < 4; ++vg) {
                        const u32x4 sp = meta[16 + 2 * vg + g];
                        const u32x4 ep = meta[24 + 2 * vg + g];
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const bool vis = kv_valid && my_kv >= (int)sp[r] && my_kv < (int)ep[r];
                            s[4 * vg + r] = vis ? s[4 * vg + r] : 0.f;
                        }
                    }
                }
            } else if (TAIL) {
#pragma unroll
                for (int v = 0; v < 16; ++v) s[v] = kv_valid ? s[v] : 0.f;
            }
            u32x4 pu[2];
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e) pu[j][e] = E::pack(s[8 * j + 2 * e], s[8 * j + 2 * e + 1]);
            *reinterpret_cast<u32x4*>(pbuf + pb_off) = pu[0];
            *reinterpret_cast<u32x4*>(pbuf + pb_off + 64 * 8) = pu[1];
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const u32x4 a = {da[dt][j][0][0], da[dt][j][0][1], da[dt][j][1][0], da[dt][j][1][1]};
                    acc[dt] = E::mfma(as_bf16x8(a), as_bf16x8(pu[j]), acc[dt]);
                }
        }
        if (s_live) s_carry = s_new;
    };

    auto d_step = [&](bool pv_live, bool ds_live, const uint16_t* tile_p1, const uint16_t* tile_p2, const u32x4* meta,
                      const uint16_t* pbuf, uint16_t* dst, f32x16& dp_carry) __attribute__((always_inline)) {
        const char* dor = reinterpret_cast<const char*>(tile_p1);                    // dO rows of tile i-1
        const char* qt = reinterpret_cast<const char*>(tile_p2);                     // Q of tile i-2
        u32x4 pu[2];
        u32x2 qa[4][2][2];
        bf16x8 da[8];
        if (pv_live) {
#pragma unroll
            for (int kk = 0; kk < NKK; ++kk)
                da[kk] = *reinterpret_cast<const bf16x8*>(dor + row_rd + ((uint32_t)(kk * 32) ^ row_h));
        }
        if (ds_live) {
            pu[0] = *reinterpret_cast<const u32x4*>(pbuf + pb_off);
            pu[1] = *reinterpret_cast<const u32x4*>(pbuf + pb_off + 64 * 8);
        }
        __builtin_amdgcn_sched_barrier(0);
        f32x16 dp_new;
        if (pv_live) {
#pragma unroll
            for (int v = 0; v < 16; ++v) dp_new[v] = 0.f;
#pragma unroll
            for (int kk = 0; kk < NKK; ++kk) dp_new = E::mfma(da[kk], breg[kk], dp_new);
        }
        if (ds_live) {
            // Q^T operands: requested once the dO operands are consumed
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    qa[dt][j][0] = lds_read_tr16(reinterpret_cast<const uint16_t*>(qt + t_rd[dt][0] + j * 4096));
                    qa[dt][j][1] = lds_read_tr16(reinterpret_cast<const uint16_t*>(qt + t_rd[dt][1] + j * 4096));
                }
            u32x4 dsu[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const f32x4 da4 = __builtin_bit_cast(f32x4, meta[8 + 4 * j + g]);       // rows 16j + 4g + 0..3
                const f32x4 db4 = __builtin_bit_cast(f32x4, meta[8 + 4 * j + 2 + g]);   // rows 16j + 8 + 4g + 0..3
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    // registers 8j + 2e, 8j + 2e + 1 are rows 16j + 8(e/2) + 4g + 2(e%2) + {0, 1}
                    const float d0 = (e < 2) ? da4[2 * (e & 1)] : db4[2 * (e & 1)];
                    const float d1 = (e < 2) ? da4[2 * (e & 1) + 1] : db4[2 * (e & 1) + 1];
                    // scale * P * (dP - delta), with delta * scale from the record
                    dsu[j][e] = E::pack(E::lo(pu[j][e]) * fmaf(dp_carry[8 * j + 2 * e], p.scale, -d0),
                                          E::hi(pu[j][e]) * fmaf(dp_carry[8 * j + 2 * e + 1], p.scale, -d1));
                }
            }
            uint16_t* dsp = dst + (32 * slice + l32) * DSS + 4 * g;
#pragma unroll
            for (int vg = 0; vg < 4; ++vg) {
                const u32x2 w = {dsu[vg >> 1][2 * (vg & 1)], dsu[vg >> 1][2 * (vg & 1) + 1]};
                *reinterpret_cast<u32x2*>(dsp + 8 * vg) = w;
            }
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const u32x4 a = {qa[dt][j][0][0], qa[dt][j][0][1], qa[dt][j][1][0], qa[dt][j][1][1]};
                    acc[dt] = E::mfma(as_bf16x8(a), as_bf16x8(dsu[j]), acc[dt]);
                }
        }
        if (pv_live) dp_carry = dp_new;
    };

    // The loop exists once per role (no branch on the role inside it).
    auto run = [&](auto tail_c, auto role_c) {
        constexpr bool DROLE = decltype(role_c)::value;
        if (n_iter == 0) return;
        // tile i lives in qt(i % 6) / dot(i % 6) with its row metadata in meta_s4[i % 6]; P(i) in pbf(i & 1); dS^T(i) in dst(i & 1)
        auto qt = [&](int k) { return smem + OFF_Q + k * TILE_ELEMS; };
        auto dot = [&](int k) { return smem + OFF_DO + k * TILE_ELEMS; };
        auto dst = [&](int k) { return smem + OFF_DST + k * DST_ELEMS; };
        auto pbf = [&](int k) { return smem + OFF_PB + k * PB_ELEMS; };
        auto m6 = [](int x) { return x >= NQD ? x - NQD : x; };
        // dS^T workspace offsets of the tiles in flight: a tile enters at [5] when requested
        // (two steps ahead); at step i (before that step's shift) tile i is at [3], tile i-3 at [0]
        int64_t w_q[6] = {0, 0, 0, 0, 0, 0};
        int64_t b_q[6] = {0, 0, 0, 0, 0, 0};    // BIAS: offset of (b, h, first row of the tile) in the bias
        int r_q[6] = {0, 0, 0, 0, 0, 0};        // BIAS: first row of the tile
        auto fetch = [&](int buf) {   // start the loads of the next tile of the walk
            w_q[5] = ws_head + (int64_t)cur_qt * (BN * BM);
            if (BIAS) {
                r_q[5] = p.row_begin + cur_qt * BM;
                b_q[5] = b * p.bias_b + (hk * p.G + cur_gi) * p.bias_h + (int64_t)r_q[5] * p.bias_r;
            }
            if (!DROLE) prefetch(buf);
            advance();
        };
        auto shift = [&]() {
#pragma unroll
            for (int k = 0; k < 5; ++k) {
                w_q[k] = w_q[k + 1];
                if (BIAS) { b_q[k] = b_q[k + 1]; r_q[k] = r_q[k + 1]; }
            }
        };
        f32x16 carry;     // P-wave: raw S of the previous tile; D-wave: dP of the previous tile
#pragma unroll
        for (int v = 0; v < 16; ++v) carry[v] = 0.f;
        int rc = 0;       // i % 6

        auto step = [&](int i, bool s_live, bool pv_live, bool ds_live, bool copy) __attribute__((always_inline)) {
            // A P-wave's part of tile i (requested two steps ago) must have landed.  Vector-memory
            // operations complete in issue order, and after the loads of tile i the wave has issued
            // at least: the 4 loads of tile i+1 (requested in step i-1, or in the prologue), and
            // from step 5 on also the 2 dS^T stores of step i-2 and the 2 of step i-1 (steps 0-2
            // store nothing; wave 0's metadata loads and the bias loads only add to this).  So "at
            // most 8 outstanding" (4 in the first steps) says tile i is there and leaves everything
            // younger in flight.
            if (!DROLE) {
                if (i + 1 >= n_iter) wait_vmcnt<0>();
                else if (i >= 5) wait_vmcnt<8>();
                else wait_vmcnt<4>();
            }
            lds_barrier();
            // tile i+2 replaces tile i-4, whose last readers finished long before this barrier
            if (i + 2 < n_iter) fetch(m6(rc + 2));
            const int r1 = m6(rc + 5), r2 = m6(rc + 4);     // (i - 1) % 6, (i - 2) % 6
            if (!DROLE)
                p_step(tail_c, s_live, pv_live, qt(rc), dot(r1), meta_s4[r1], pbf((i + 1) & 1), carry, b_q[2], r_q[2]);
            else
                d_step(pv_live, ds_live, dot(r1), qt(r2), meta_s4[r2], pbf(i & 1), dst(i & 1), carry);
            // dS^T(i-3) to HBM last: its LDS read queues behind this step's operand reads
            // instead of delaying them, and only has to finish before the next barrier
            if (!DROLE && copy) copy_out(dst((i + 1) & 1), w_q[0]);
            shift();
            rc = m6(rc + 1);
        };
        fetch(0);
        shift();
        if (n_iter > 1) fetch(1);
        shift();
        const int last = n_iter + 1;
        int i = 0;
        for (; i < 3 && i <= last; ++i) step(i, i < n_iter, i >= 1 && i <= n_iter, i >= 2, false);
        // Steady state of the plain bf16 kernel: steps 3 .. 3 + 6 trips - 1 (every one of them with all
        // its parts alive and a tile to request) run in the hand-scheduled loops of gen_bwd_loop.py,
        // six steps a trip; the steps after them continue below as if they had run here.
        if constexpr (DH == 128 && !MASKED && !BIAS && !F16 && !decltype(tail_c)::value) {
            int trips = uniform32((n_iter - 5) / 6);
            if (i == 3 && trips >= 1 && (p.row_end - p.row_begin) % BM == 0) {
                const int steps = 6 * trips;
                uint32_t ra[8], ta[8];
#pragma unroll
                for (int kk = 0; kk < 8; ++kk)
                    ra[kk] = lds0 + (DROLE ? OFF_DO : OFF_Q) * 2 + row_rd + ((uint32_t)(kk * 32) ^ row_h);
#pragma unroll
                for (int dt = 0; dt < 4; ++dt) {
                    ta[2 * dt] = lds0 + (DROLE ? OFF_Q : OFF_DO) * 2 + t_rd[dt][0];
                    ta[2 * dt + 1] = lds0 + (DROLE ? OFF_Q : OFF_DO) * 2 + t_rd[dt][1];
                }
                const uint32_t a_pb = lds0 + OFF_PB * 2 + (uint32_t)pb_off * 2;
                const uint32_t a_meta = meta0 + (uint32_t)g * 16u;
                if constexpr (!DROLE) {
                    uint16_t* ws_k = p.ds_ws + (int64_t)kblk * p.ws_ld;
                    const char* qp = uniform_ptr(q_head + (int64_t)(p.row_begin + cur_qt * BM) * qrow_b);
                    const char* dop = uniform_ptr(do_head + (int64_t)(p.row_begin + cur_qt * BM) * dorow_b);
                    const char* mp = uniform_ptr(reinterpret_cast<const char*>(meta_head + cur_qt * 64));
                    const char* wn = uniform_ptr(reinterpret_cast<const char*>(ws_k + ws_head + (int64_t)cur_qt * (BN * BM)));
                    const char* w0 = uniform_ptr(reinterpret_cast<const char*>(ws_k + w_q[0]));
                    const char* w1 = uniform_ptr(reinterpret_cast<const char*>(ws_k + w_q[1]));
                    const char* w2 = uniform_ptr(reinterpret_cast<const char*>(ws_k + w_q[2]));
                    const char* w3 = uniform_ptr(reinterpret_cast<const char*>(ws_k + w_q[3]));
                    const char* w4 = uniform_ptr(reinterpret_cast<const char*>(ws_k + w_q[4]));
                    const char* w5 = w4;
                    int left = uniform32(cur_left);
                    const int64_t hdq = uniform64((int64_t)p.qs.h * 2 - (int64_t)n_qtiles * BM * qrow_b);
                    const int64_t hddo = uniform64((int64_t)p.dos.h * 2 - (int64_t)n_qtiles * BM * dorow_b);
                    const int64_t hdws = uniform64((int64_t)p.ws_bh * 2 - (int64_t)n_qtiles * (BN * BM * 2));
                    const uint32_t a_cp = lds0 + OFF_DST * 2 + (uint32_t)(cp_token * DSS + cp_part * 8) * 2;
                    const uint32_t g_cp0 = (uint32_t)(cp_token * BM + cp_part * 8) * 2, g_cp1 = g_cp0 + 64 * BM * 2;
                    const uint32_t lr = (uint32_t)(lane >> 4) + 8u * slice;
                    const uint32_t g_q0 = lr * qrow_b + ld_c0, g_q1 = (lr + 4) * qrow_b + ld_c1;
                    const uint32_t g_d0 = lr * dorow_b + ld_c0, g_d1 = (lr + 4) * dorow_b + ld_c1;
                    wait_vmcnt<4>();    // tile 3 (the loads of tile 4 may be in flight); the loop counts from there
                    asm volatile(
#include "lvx_bwd_loop_p.inc"
                        : "+{v[0:15]}"(acc[0]), "+{v[16:31]}"(acc[1]), "+{v[32:47]}"(acc[2]), "+{v[48:63]}"(acc[3]),
                          "+{v[96:111]}"(carry), "+{s[44:45]}"(qp), "+{s[46:47]}"(dop), "+{s[48:49]}"(mp), "+{s[50:51]}"(wn),
                          "+{s52}"(left), "+{s64}"(trips), "+{s[66:67]}"(w0), "+{s[68:69]}"(w1), "+{s[70:71]}"(w2),
                          "+{s[72:73]}"(w3), "+{s[74:75]}"(w4), "+{s[76:77]}"(w5)
                        : "{v[64:67]}"(breg[0]), "{v[68:71]}"(breg[1]), "{v[72:75]}"(breg[2]), "{v[76:79]}"(breg[3]),
                          "{v[80:83]}"(breg[4]), "{v[84:87]}"(breg[5]), "{v[88:91]}"(breg[6]), "{v[92:95]}"(breg[7]),
                          "{v200}"(ra[0]), "{v201}"(ra[1]), "{v202}"(ra[2]), "{v203}"(ra[3]),
                          "{v204}"(ra[4]), "{v205}"(ra[5]), "{v206}"(ra[6]), "{v207}"(ra[7]),
                          "{v208}"(ta[0]), "{v209}"(ta[1]), "{v210}"(ta[2]), "{v211}"(ta[3]),
                          "{v212}"(ta[4]), "{v213}"(ta[5]), "{v214}"(ta[6]), "{v215}"(ta[7]),
                          "{v216}"(a_pb), "{v217}"(a_meta), "{v218}"(a_cp), "{v219}"(g_cp0), "{v220}"(g_cp1),
                          "{v221}"(g_q0), "{v222}"(g_q1), "{v223}"(g_d0), "{v224}"(g_d1), "{v225}"((uint32_t)lane * 4u),
                          "{s40}"(uniform32(c)), "{s41}"(uniform32((uint32_t)BM * qrow_b)), "{s42}"(uniform32((uint32_t)BM * dorow_b)), "{s53}"(uniform32(n_qtiles)),
                          "{s[54:55]}"(hdq), "{s[56:57]}"(hddo), "{s[60:61]}"(hdws),
                          "{s62}"(uniform32(lds0 + (uint32_t)slice * 2048u)), "{s63}"(uniform32(meta0)), "{s65}"(uniform32(wave == 0 ? 1 : 0))
                        : "memory", "vcc", "scc", "m0", "s78", "s79", LVX_BWD_LOOP_CLOBBERS);
                    wait_vmcnt<0>();    // the steps below count the operations in flight from scratch
                    w_q[0] = reinterpret_cast<const uint16_t*>(w0) - ws_k;
                    w_q[1] = reinterpret_cast<const uint16_t*>(w1) - ws_k;
                    w_q[2] = reinterpret_cast<const uint16_t*>(w2) - ws_k;
                    w_q[3] = reinterpret_cast<const uint16_t*>(w3) - ws_k;
                    w_q[4] = reinterpret_cast<const uint16_t*>(w4) - ws_k;
                } else {
                    const uint32_t a_ds = lds0 + OFF_DST * 2 + (uint32_t)((32 * slice + l32) * DSS + 4 * g) * 2;
                    asm volatile(
#include "lvx_bwd_loop_d.inc"
                        : "+{v[0:15]}"(acc[0]), "+{v[16:31]}"(acc[1]), "+{v[32:47]}"(acc[2]), "+{v[48:63]}"(acc[3]),
                          "+{v[96:111]}"(carry), "+{s64}"(trips)
                        : "{v[64:67]}"(breg[0]), "{v[68:71]}"(breg[1]), "{v[72:75]}"(breg[2]), "{v[76:79]}"(breg[3]),
                          "{v[80:83]}"(breg[4]), "{v[84:87]}"(breg[5]), "{v[88:91]}"(breg[6]), "{v[92:95]}"(breg[7]),
                          "{v200}"(ra[0]), "{v201}"(ra[1]), "{v202}"(ra[2]), "{v203}"(ra[3]),
                          "{v204}"(ra[4]), "{v205}"(ra[5]), "{v206}"(ra[6]), "{v207}"(ra[7]),
                          "{v208}"(ta[0]), "{v209}"(ta[1]), "{v210}"(ta[2]), "{v211}"(ta[3]),
                          "{v212}"(ta[4]), "{v213}"(ta[5]), "{v214}"(ta[6]), "{v215}"(ta[7]),
                          "{v216}"(a_pb), "{v217}"(a_meta), "{v218}"(a_ds), "{s40}"(uniform32(p.scale))
                        : "memory", "vcc", "scc", LVX_BWD_LOOP_CLOBBERS, "v219", "v220", "v221", "v222");
                }
                i += steps;
                // the walk stands at the tile after the last one requested
                const int pos = it_lo + i + 2;
                cur_gi = pos / n_live;
                cur_qt = pos % n_live;
                cur_left = n_live - cur_qt;
                if (cur_gi >= p.G) cur_gi = 0;
                enter_head();
            }
        }
        for (; i < n_iter; ++i) step(i, true, true, true, true);
        for (; i <= last; ++i) step(i, false, i <= n_iter, true, true);
        __syncthreads();
        if (!DROLE) copy_out(dst((n_iter - 1) & 1), w_q[0]);
    };
    if (d_role) {
        if (tail_block) run(std::true_type{}, std::true_type{});
        else run(std::false_type{}, std::true_type{});
    } else {
        if (tail_block) run(std::true_type{}, std::false_type{});
        else run(std::false_type{}, std::false_type{});
    }

    // ---- epilogue: rows of acc = head-dim, cols = this wave's tokens; P-waves hold dV^T, D-waves dK^T
    if (dkv_mode == 2) {
        // Several work-groups (ranges of steps) share this token block: add with
        // atomics.  The accumulator has tokens along the lanes; it is turned
        // through LDS so that each atomic instruction covers 64 consecutive
        // floats (two full lines) of one token row.
        __syncthreads();   // the staging buffers are free now
        if (n_iter > 0) {
            float* ep = reinterpret_cast<float*>(smem) + wave * (32 * EPS);
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int v = 0; v < 16; ++v) ep[l32 * EPS + dt * 32 + acc_row(v, g)] = acc[dt][v];
            __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): this wave's LDS writes have landed
            const Strides3 os = d_role ? p.dks : p.dvs;
            float* obase = reinterpret_cast<float*>(d_role ? p.dk : p.dv) + b * os.b + hk * os.h;
            for (int t = 0; t < 32; ++t) {
                const int token = kvb + 32 * slice + t;
                if (token >= p.Lkv) break;
                float* op = obase + (int64_t)token * os.s;
                if (DH >= 64 || lane < DH) unsafeAtomicAdd(op + lane, ep[t * EPS + lane]);
                if (DH == 128) unsafeAtomicAdd(op + 64 + lane, ep[t * EPS + 64 + lane]);
            }
        }
    } else if (my_kv < p.Lkv) {
        const Strides3 os = alone ? (d_role ? p.dks_whole : p.dvs_whole) : (d_role ? p.dks : p.dvs);
        void* optr = alone ? (d_role ? p.dk_whole : p.dv_whole) : (d_role ? p.dk : p.dv);
        const int64_t off = b * os.b + hk * os.h + (int64_t)my_kv * os.s;
        if (dkv_mode == 1) {
            float* op = reinterpret_cast<float*>(optr) + off;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int vg = 0; vg < 4; ++vg) {
                    const int d = dt * 32 + 8 * vg + 4 * g;
                    if (d >= DH) continue;      // only with DH = 16
                    f32x4 a = *reinterpret_cast<f32x4*>(op + d);
#pragma unroll
                    for (int r = 0; r < 4; ++r) a[r] += acc[dt][4 * vg + r];
                    *reinterpret_cast<f32x4*>(op + d) = a;
                }
        } else {
            uint16_t* op = reinterpret_cast<uint16_t*>(optr) + off;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int vg = 0; vg < 4; ++vg) {
                    const int d = dt * 32 + 8 * vg + 4 * g;
                    if (d >= DH) continue;      // only with DH = 16
                    u32x2 a;
                    a[0] = E::pack(acc[dt][4 * vg], acc[dt][4 * vg + 1]);
                    a[1] = E::pack(acc[dt][4 * vg + 2], acc[dt][4 * vg + 3]);
                    *reinterpret_cast<u32x2*>(op + d) = a;
                }
        }
    }
}

}  // namespace

namespace {
template <int DH, bool F16>
hipError_t launch_bwd_t(const BwdParams& p, bool masked, hipStream_t st) {
    const int grid = 8 * (p.whole_blocks + p.mid_blocks * p.q_splits +
                          (p.blocks_per_xcd - p.whole_blocks - p.mid_blocks) * p.q_splits2);
    if (p.bias) {
        if (masked) return launch1((bwd_kernel<DH, true, true, F16>), dim3(grid), dim3(NT), st, p);
        else return launch1((bwd_kernel<DH, false, true, F16>), dim3(grid), dim3(NT), st, p);
    } else {
        if (masked) return launch1((bwd_kernel<DH, true, false, F16>), dim3(grid), dim3(NT), st, p);
        else return launch1((bwd_kernel<DH, false, false, F16>), dim3(grid), dim3(NT), st, p);
    }
}
}  // namespace

hipError_t launch_bwd(const BwdParams& p, bool masked, hipStream_t st) {
    switch (p.D) {
        case 16: return p.f16 ? launch_bwd_t<16, true>(p, masked, st) : launch_bwd_t<16, false>(p, masked, st);
        case 32: return p.f16 ? launch_bwd_t<32, true>(p, masked, st) : launch_bwd_t<32, false>(p, masked, st);
        case 64: return p.f16 ? launch_bwd_t<64, true>(p, masked, st) : launch_bwd_t<64, false>(p, masked, st);
        case 128: return p.f16 ? launch_bwd_t<128, true>(p, masked, st) : launch_bwd_t<128, false>(p, masked, st);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace lvx
