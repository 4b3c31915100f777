// Cross-attention backward for gfx950 from the saved LSE and delta:
//   P = exp(scale*Q K^T - LSE);  dV = P^T dO;  dP = dO V^T;
//   dS = P * (dP - delta);  dK = scale * dS^T Q;  dQ = scale * dS K.
//
// Mapping.  A work-group (4 waves, one per SIMD) owns a block of 128 visual
// tokens of one kv head and streams every text row of the window for every q
// head of the GQA group past it, 32 rows at a time.  Wave w owns tokens
// 32w..32w+31 of the block: its K and V rows sit in registers as MFMA B
// operands for the whole kernel, and its dK^T / dV^T (128 x 32 each, fp32) stay
// in accumulators until the end, so the sum over the q heads of the group and
// over all rows never leaves the register file.
//
// dQ = scale * dS K sums over ALL tokens, i.e. over every work-group of the kv
// head.  Adding 51 partial tiles per row with fp32 atomics costs more than the
// whole rest of the kernel on this machine (atomic adds sustain about 1.3 TB/s),
// so dQ is not formed here: the waves gather scale*dS (bf16) in LDS and stream
// it to a workspace dS^T[b, h, token, row] in HBM with full 64-byte segments,
// and a batched GEMM (launched by the caller right after) contracts it with K.
// The workspace costs 2 bytes per (row, token, head) written once and read once.
//
// Per 32-row step and wave (all MFMA are 32x32x16 bf16):
//   (1) S, dP        2 x 8 MFMA   A = Q / dO rows from LDS (16-byte reads)
//   (2) P, dS        VALU only    exp2, the two multiplies, bf16 packing
//   (3) dV^T, dK^T   2 x 8 MFMA   A = dO^T / Q^T, read from the SAME row-major
//                                 LDS tiles with the transposing LDS read; B =
//                                 P / dS straight from the registers of (2)
//   (4) dS^T store   LDS -> HBM   the [128 tokens][32 rows] tile the waves wrote
// With one wave per SIMD nothing else hides the VALU work of (2), so the loop is
// software-pipelined: the body of step i runs (1) and (2) of tile i together
// with (3) and (4) of tile i-1, which are independent of them.  Q/dO tiles are
// triple-buffered in LDS and the dS^T tile and row metadata double-buffered, so
// one barrier per step is enough.
#include <type_traits>

#include "lvx_common.hpp"
#include "lvx_kernels.hpp"

namespace lvx {

namespace {

constexpr int D = 128;
constexpr int BN = 128;       // visual tokens per work-group
constexpr int BM = 32;        // text rows per step
// Every Q / dO tile is staged twice, because no single row stride serves both
// access patterns without bank conflicts: 16-byte row reads want 16 consecutive
// rows on 16 distinct bank quads (68-dword rows), a transposing read touches 8
// rows x 16 dwords and wants them to tile the 64 banks twice (72-dword rows).
constexpr int QS = D + 8;     // row stride of the copy read by rows      (stage 1)
constexpr int QT = D + 16;    // row stride of the copy read transposed   (stage 3)
constexpr int DSS = BM + 8;   // row stride of the dS^T tile [token][row] (80 bytes, 16-byte aligned rows)

constexpr int QD_ELEMS = 2 * BM * QS + 2 * BM * QT;   // one (Q, dO) tile pair, both copies
constexpr int OFF_T = 2 * BM * QS;                   // transposed-read copies inside a pair
constexpr int DST_ELEMS = BN * DSS;            // one dS^T tile
constexpr int OFF_QD = 0;
constexpr int OFF_DST = OFF_QD + 3 * QD_ELEMS;
constexpr int SMEM_ELEMS = OFF_DST + 2 * DST_ELEMS;

constexpr float LOG2E = 1.4426950408889634f;

template <bool MASKED>
__global__ __launch_bounds__(256, 1) void bwd_kernel(const BwdParams p) {
    __shared__ __attribute__((aligned(16))) uint16_t smem[SMEM_ELEMS];
    // per-row metadata of a staged tile, double-buffered: 8 x 16 bytes each of
    // LSE*log2e, delta, kv_start, kv_end
    __shared__ u32x4 meta_s4[2][BM];

    const int wid = xcd_remap(blockIdx.x, p.total_wg);
    if (wid >= p.total_wg) return;
    const int kblk = wid % p.n_kv_blocks;
    const int bh = wid / p.n_kv_blocks;
    const int hk = bh % p.Hkv;
    const int b = bh / p.Hkv;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, l32 = lane & 31, g = lane >> 5;

    int kv_len = p.Lkv;
    if (p.kv_len) kv_len = min(p.kv_len[b], p.Lkv);
    const int kvb = kblk * BN;
    const int my_kv = kvb + 32 * wave + l32;
    const bool kv_valid = my_kv < kv_len;
    const bool tail_block = kvb + BN > kv_len;

    const uint16_t* kbase = p.k + b * p.ks.b + hk * p.ks.h;
    const uint16_t* vbase = p.v + b * p.vs.b + hk * p.vs.h;

    // ---- prologue: K, V rows of this wave as B operands (contraction over d)
    bf16x8 kreg[8], vreg[8];
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
        kreg[kk] = as_bf16x8(ldg16(kbase + (int64_t)my_kv * p.ks.s + kk * 16 + g * 8, kv_valid));
        vreg[kk] = as_bf16x8(ldg16(vbase + (int64_t)my_kv * p.vs.s + kk * 16 + g * 8, kv_valid));
    }

    f32x16 dk[4], dv[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) { dk[dt][v] = 0.f; dv[dt][v] = 0.f; }

    const int n_qtiles = (p.row_end - p.row_begin + BM - 1) / BM;
    const int n_iter = (kvb < kv_len) ? p.G * n_qtiles : 0;
    const float c = p.scale_log2e;

    // staging role of this thread: threads 0..127 carry Q, 128..255 carry dO
    const int st = tid & 127;
    const int s_chunk = st & 15, s_group = st >> 4;
    const bool is_do = tid >= 128;
    const int stage_off = (is_do ? BM * QS : 0) + 4 * s_group * QS + s_chunk * 8;
    const int stage_off_t = OFF_T + (is_do ? BM * QT : 0) + 4 * s_group * QT + s_chunk * 8;
    const uint16_t* g_base = is_do ? p.dout + b * p.dos.b : p.q + b * p.qs.b;
    const int64_t g_hs = is_do ? p.dos.h : p.qs.h;
    const int g_rs = (int)(is_do ? p.dos.s : p.qs.s);
    const int meta_kind = (tid >> 5) & 3;    // 0 LSE, 1 delta, 2 kv_start, 3 kv_end
    const uint32_t* m_base = reinterpret_cast<const uint32_t*>(p.lse);
    int64_t m_hs = p.Lq;
    if (meta_kind == 1) m_base = reinterpret_cast<const uint32_t*>(p.delta);
    if (MASKED && meta_kind >= 2) {
        m_base = reinterpret_cast<const uint32_t*>(meta_kind == 2 ? p.kv_start : p.kv_end) + (int64_t)b * p.Lq;
        m_hs = 0;
    } else {
        m_base += (int64_t)b * p.Hq * p.Lq;
    }

    // per-lane offset of the transposing operand reads (Q^T / dO^T, rows in accumulator order)
    const int off_qT = OFF_T + tr_lane_offset(lane, QT, true);
    // dS^T copy-out: 512 chunks of 16 bytes per tile, two per thread
    const int cp_token = tid >> 2, cp_part = tid & 3;
    uint16_t* ws_lane = p.ds_ws + ((int64_t)kvb + cp_token) * p.ws_ld + cp_part * 8;

    // token blocks of one kv head walk the (head, row tile) list from different
    // starting points, which spreads their reads of Q / dO over the L2
    int cur_gi = 0, cur_qt = 0;
    if (n_iter > 0) {
        const int it_shift = (int)(((int64_t)kblk * 7) % n_iter);
        cur_gi = it_shift / n_qtiles;
        cur_qt = it_shift % n_qtiles;
    }

    // Every load is unconditional: rows past the window are clamped to its last
    // row (their LSE is forced to +inf, so P = 0 and nothing they carry reaches a
    // result), and the fetch after the last tile re-reads some tile.
    u32x4 pre[4];
    uint32_t pre_m = 0;
    bool pre_ok = false;
    auto prefetch = [&]() {
        const int h = hk * p.G + cur_gi;
        const int r0 = p.row_begin + cur_qt * BM;
        const uint16_t* base = g_base + h * g_hs + s_chunk * 8;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = min(r0 + 4 * s_group + i, p.row_end - 1);
            pre[i] = *reinterpret_cast<const u32x4*>(base + row * g_rs);
        }
        const int mrow = r0 + (tid & 31);
        pre_ok = mrow < p.row_end;
        pre_m = m_base[h * m_hs + min(mrow, p.row_end - 1)];   // used one step later
    };
    auto advance = [&]() {   // next (head, row tile) of the walk, wrapping
        if (++cur_qt == n_qtiles) {
            cur_qt = 0;
            if (++cur_gi == p.G) cur_gi = 0;
        }
    };

    auto stage_write = [&](uint16_t* qd, u32x4* meta) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<u32x4*>(qd + stage_off + i * QS) = pre[i];
            *reinterpret_cast<u32x4*>(qd + stage_off_t + i * QT) = pre[i];
        }
        const float l = __uint_as_float(pre_m);
        // exp2(x - inf) = 0: rows that saw no key (or do not exist) get P = 0
        const float lt = (!pre_ok || l == -INFINITY) ? INFINITY : l * LOG2E;
        const uint32_t m = meta_kind == 0 ? __float_as_uint(lt) : (pre_ok ? pre_m : 0u);
        reinterpret_cast<uint32_t*>(meta)[tid & 127] = m;   // both halves write the same words
    };

    // (1) S = Q K_w^T, dP = dO V_w^T : rows = text rows, cols = this wave's tokens
    auto stage1 = [&](const uint16_t* qd, f32x16& s, f32x16& dp) {
        const uint16_t* qrow = qd + l32 * QS + g * 8;
#pragma unroll
        for (int v = 0; v < 16; ++v) { s[v] = 0.f; dp[v] = 0.f; }
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            const bf16x8 aq = *reinterpret_cast<const bf16x8*>(qrow + kk * 16);
            const bf16x8 ad = *reinterpret_cast<const bf16x8*>(qrow + BM * QS + kk * 16);
            s = mfma32(aq, kreg[kk], s);
            dp = mfma32(ad, vreg[kk], dp);
        }
    };

    // (2) P and scale*dS as bf16 B operands (register v of lane-half g is text
    //     row 8*(v/4)+4g+(v%4)), and scale*dS handed to the other waves as
    //     dST[token of the block][text row]
    auto stage2 = [&](auto tail_c, f32x16& s, f32x16& dp, const u32x4* meta, uint16_t* dst, bf16x8 pb[2],
                      bf16x8 dsb[2]) {
        constexpr bool TAIL = decltype(tail_c)::value;
#pragma unroll
        for (int vg = 0; vg < 4; ++vg) {
            const f32x4 l4 = __builtin_bit_cast(f32x4, meta[2 * vg + g]);
            const f32x4 d4 = __builtin_bit_cast(f32x4, meta[8 + 2 * vg + g]);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int v = 4 * vg + r;
                const float pv = __builtin_amdgcn_exp2f(fmaf(s[v], c, -l4[r]));
                s[v] = pv;
                dp[v] = pv * p.scale * (dp[v] - d4[r]);
            }
        }
        if (MASKED) {
#pragma unroll
            for (int vg = 0; vg < 4; ++vg) {
                const u32x4 sp = meta[16 + 2 * vg + g];
                const u32x4 ep = meta[24 + 2 * vg + g];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const bool vis = kv_valid && my_kv >= (int)sp[r] && my_kv < (int)ep[r];
                    s[4 * vg + r] = vis ? s[4 * vg + r] : 0.f;
                    dp[4 * vg + r] = vis ? dp[4 * vg + r] : 0.f;
                }
            }
        } else if (TAIL) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                s[v] = kv_valid ? s[v] : 0.f;
                dp[v] = kv_valid ? dp[v] : 0.f;
            }
        }
        u32x4 dsu[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            u32x4 u;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                u[e] = pack_bf16(s[8 * j + 2 * e], s[8 * j + 2 * e + 1]);
                dsu[j][e] = pack_bf16(dp[8 * j + 2 * e], dp[8 * j + 2 * e + 1]);
            }
            pb[j] = as_bf16x8(u);
            dsb[j] = as_bf16x8(dsu[j]);
        }
        uint16_t* dsp = dst + (32 * wave + l32) * DSS + 4 * g;
#pragma unroll
        for (int vg = 0; vg < 4; ++vg) {
            const u32x2 w = {dsu[vg >> 1][2 * (vg & 1)], dsu[vg >> 1][2 * (vg & 1) + 1]};
            *reinterpret_cast<u32x2*>(dsp + 8 * vg) = w;
        }
    };

    // (3) dV_w^T += dO^T P,  dK_w^T += Q^T (scale*dS)  (contraction over the 32 text rows)
    auto stage3 = [&](const uint16_t* qd, const bf16x8 pb[2], const bf16x8 dsb[2]) {
        const uint16_t* qt = qd + off_qT;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const bf16x8 a1 = lds_operand_tr(qt + BM * QT + 16 * j * QT + dt * 32, 8 * QT);
                const bf16x8 a2 = lds_operand_tr(qt + 16 * j * QT + dt * 32, 8 * QT);
                dv[dt] = mfma32(a1, pb[j], dv[dt]);
                dk[dt] = mfma32(a2, dsb[j], dk[dt]);
            }
    };

    // (4) the finished dS^T tile goes to HBM: dS^T[b, h, token, row - row_begin]
    auto stage4 = [&](const uint16_t* dst, int h, int r0) {
        uint16_t* gp = ws_lane + ((int64_t)b * p.Hq + h) * p.ws_bh + (r0 - p.row_begin);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const u32x4 w = *reinterpret_cast<const u32x4*>(dst + (cp_token + 64 * j) * DSS + cp_part * 8);
#ifdef LVX_EXP_NOSTORE
            if (w[0] == 0x12345678u)
#endif
            *reinterpret_cast<u32x4*>(gp + (int64_t)64 * j * p.ws_ld) = w;
        }
    };

    auto run = [&](auto tail_c) {
        if (n_iter == 0) return;
        uint16_t* qd0 = smem + OFF_QD;                 // tile being staged / used by (1),(2)
        uint16_t* qd1 = smem + OFF_QD + QD_ELEMS;      // next to be staged
        uint16_t* qd2 = smem + OFF_QD + 2 * QD_ELEMS;  // previous tile, used by (3)
        uint16_t* ds0 = smem + OFF_DST;
        uint16_t* ds1 = smem + OFF_DST + DST_ELEMS;
        int mb = 0;

        bf16x8 pb[2], dsb[2];
        f32x16 s, dp;
        int h_prev, r0_prev;          // tile whose (3), (4) run in the current step

        // ---- first tile: (1), (2) only
        prefetch();
        h_prev = hk * p.G + cur_gi;
        r0_prev = p.row_begin + cur_qt * BM;
        advance();
        stage_write(qd0, meta_s4[0]);
        __syncthreads();
        prefetch();
        stage1(qd0, s, dp);
        stage2(tail_c, s, dp, meta_s4[0], ds0, pb, dsb);

        // ---- steady state: (1), (2) of tile i with (3), (4) of tile i-1
        for (int i = 1; i < n_iter; ++i) {
            { uint16_t* t = qd2; qd2 = qd0; qd0 = qd1; qd1 = t; }   // rotate tile buffers
            { uint16_t* t = ds0; ds0 = ds1; ds1 = t; }              // ds1 = dS^T of tile i-1
            mb ^= 1;
            const int h_cur = hk * p.G + cur_gi;
            const int r0_cur = p.row_begin + cur_qt * BM;
            advance();
            stage_write(qd0, meta_s4[mb]);
            __syncthreads();
            // stores of the finished tile go out before this step's loads, so that
            // waiting for those loads one step later never waits for younger stores
            stage4(ds1, h_prev, r0_prev);
            prefetch();
            stage1(qd0, s, dp);
            stage3(qd2, pb, dsb);
            stage2(tail_c, s, dp, meta_s4[mb], ds0, pb, dsb);
            h_prev = h_cur;
            r0_prev = r0_cur;
        }

        // ---- drain: (3), (4) of the last tile
        __syncthreads();
        stage4(ds0, h_prev, r0_prev);
        stage3(qd0, pb, dsb);
    };
    if (tail_block) run(std::true_type{});
    else run(std::false_type{});

    // ---- epilogue: dK^T / dV^T rows = head-dim, cols = this wave's tokens
    if (my_kv < p.Lkv) {
        if (p.dkv_accumulate) {
            float* dkp = reinterpret_cast<float*>(p.dk) + b * p.dks.b + hk * p.dks.h + (int64_t)my_kv * p.dks.s;
            float* dvp = reinterpret_cast<float*>(p.dv) + b * p.dvs.b + hk * p.dvs.h + (int64_t)my_kv * p.dvs.s;
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                for (int vg = 0; vg < 4; ++vg) {
                    const int d = dt * 32 + 8 * vg + 4 * g;
                    f32x4 a = *reinterpret_cast<f32x4*>(dkp + d);
                    f32x4 bb = *reinterpret_cast<f32x4*>(dvp + d);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        a[r] += dk[dt][4 * vg + r];
                        bb[r] += dv[dt][4 * vg + r];
                    }
                    *reinterpret_cast<f32x4*>(dkp + d) = a;
                    *reinterpret_cast<f32x4*>(dvp + d) = bb;
                }
        } else {
            uint16_t* dkp = reinterpret_cast<uint16_t*>(p.dk) + b * p.dks.b + hk * p.dks.h + (int64_t)my_kv * p.dks.s;
            uint16_t* dvp = reinterpret_cast<uint16_t*>(p.dv) + b * p.dvs.b + hk * p.dvs.h + (int64_t)my_kv * p.dvs.s;
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                for (int vg = 0; vg < 4; ++vg) {
                    const int d = dt * 32 + 8 * vg + 4 * g;
                    u32x2 a, bb;
                    a[0] = pack_bf16(dk[dt][4 * vg], dk[dt][4 * vg + 1]);
                    a[1] = pack_bf16(dk[dt][4 * vg + 2], dk[dt][4 * vg + 3]);
                    bb[0] = pack_bf16(dv[dt][4 * vg], dv[dt][4 * vg + 1]);
                    bb[1] = pack_bf16(dv[dt][4 * vg + 2], dv[dt][4 * vg + 3]);
                    *reinterpret_cast<u32x2*>(dkp + d) = a;
                    *reinterpret_cast<u32x2*>(dvp + d) = bb;
                }
        }
    }
}

}  // namespace

hipError_t launch_bwd(const BwdParams& p, bool masked, hipStream_t st) {
    const int grid = ((p.total_wg + 7) / 8) * 8;
    if (masked)
        hipLaunchKernelGGL(bwd_kernel<true>, dim3(grid), dim3(256), 0, st, p);
    else
        hipLaunchKernelGGL(bwd_kernel<false>, dim3(grid), dim3(256), 0, st, p);
    return hipGetLastError();
}

}  // namespace lvx
