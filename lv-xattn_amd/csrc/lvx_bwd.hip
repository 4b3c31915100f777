// Cross-attention backward for gfx950 from the saved LSE and delta:
//   P = exp(scale*Q K^T - LSE);  dV = P^T dO;  dP = dO V^T;
//   dS = P * (dP - delta);  dK = scale * dS^T Q;  dQ = scale * dS K.
//
// Mapping.  A work-group (4 waves) owns a block of 128 visual tokens of one kv
// head and streams every text row of the window for every q head of the GQA
// group past it, 32 rows at a time.  Wave w owns tokens 32w..32w+31 of the
// block: its K and V rows sit in registers as MFMA B operands for the whole
// kernel, and its dK^T / dV^T (128 x 32 each, fp32) stay in accumulators until
// the end, so the sum over the q heads of the group and over all rows never
// leaves the register file.  dQ needs all 128 tokens of the block: the waves
// exchange dS (bf16) through LDS, wave w then forms dQ for head-dim columns
// 32w..32w+31 with the matching K slice held in registers, and adds it to the
// fp32 dQ accumulator in HBM with atomic adds (other token blocks add to the
// same rows).  The dQ tile is produced with the head-dim along the lanes, so an
// atomic instruction covers whole 128-byte lines.
//
// Per 32-row step and wave: S and dP (2 x 8 MFMA, A = Q / dO row-major from
// LDS), dV^T and dK^T (2 x 8 MFMA, A = dO^T / Q^T from LDS, B = P / dS straight
// from the accumulators; the transposed tiles are staged with the row index
// permuted to match), dQ (8 MFMA).  All MFMA are 32x32x16 bf16.
#include "lvx_common.hpp"
#include "lvx_kernels.hpp"

namespace lvx {

namespace {

constexpr int D = 128;
constexpr int BN = 128;       // visual tokens per work-group
constexpr int BM = 32;        // text rows per step
constexpr int QS = D + 8;     // row stride of the row-major Q / dO tiles
constexpr int TS = BM + 8;    // row stride of the transposed Q^T / dO^T tiles
constexpr int DSS = BN + 8;   // row stride of the dS tile
constexpr int KTS = BN + 8;   // row stride of the K^T staging tile (prologue only)

constexpr int OFF_Q = 0;
constexpr int OFF_DO = OFF_Q + BM * QS;
constexpr int OFF_QT = OFF_DO + BM * QS;
constexpr int OFF_DOT = OFF_QT + D * TS;
constexpr int OFF_DS = OFF_DOT + D * TS;
constexpr int TILE_ELEMS = OFF_DS + BM * DSS;
static_assert(D * KTS <= OFF_DS, "K^T staging must fit under the dS tile");

template <bool MASKED>
__global__ __launch_bounds__(256, 1) void bwd_kernel(const BwdParams p) {
    __shared__ __attribute__((aligned(16))) uint16_t smem[TILE_ELEMS];
    __shared__ __attribute__((aligned(16))) float lse_s[BM];
    __shared__ __attribute__((aligned(16))) float delta_s[BM];
    __shared__ __attribute__((aligned(16))) int start_s[BM];
    __shared__ __attribute__((aligned(16))) int end_s[BM];

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

    uint16_t* Qs = smem + OFF_Q;
    uint16_t* dOs = smem + OFF_DO;
    uint16_t* QT = smem + OFF_QT;
    uint16_t* dOT = smem + OFF_DOT;
    uint16_t* dSs = smem + OFF_DS;

    const uint16_t* kbase = p.k + b * p.ks.b + hk * p.ks.h;
    const uint16_t* vbase = p.v + b * p.vs.b + hk * p.vs.h;

    // ---- prologue: K, V rows of this wave as B operands; K^T slice as A operand
    bf16x8 kreg[8], vreg[8], ktreg[8];
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
        kreg[kk] = as_bf16x8(ldg16(kbase + (int64_t)my_kv * p.ks.s + kk * 16 + g * 8, kv_valid));
        vreg[kk] = as_bf16x8(ldg16(vbase + (int64_t)my_kv * p.vs.s + kk * 16 + g * 8, kv_valid));
    }
    {
        // stage K^T[d][token] of the whole 128-token block (natural token order)
        uint16_t* KT = smem;
#pragma unroll
        for (int rep = 0; rep < 2; ++rep) {
            const int blk = tid + 256 * rep;        // 512 blocks of 4 tokens x 8 columns
            const int chunk = blk & 15, group = blk >> 4;
            u32x4 r[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int kv = kvb + 4 * group + i;
                r[i] = ldg16(kbase + (int64_t)kv * p.ks.s + chunk * 8, kv < kv_len);
            }
            u32x2 t8[8];
            transpose_4x8(r, t8);
#pragma unroll
            for (int d = 0; d < 8; ++d)
                *reinterpret_cast<u32x2*>(&KT[(chunk * 8 + d) * KTS + 4 * group]) = t8[d];
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 8; ++j)
            ktreg[j] = *reinterpret_cast<const bf16x8*>(&KT[(32 * wave + l32) * KTS + 16 * j + 8 * g]);
        __syncthreads();
    }

    f32x16 dk[4], dv[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) { dk[dt][v] = 0.f; dv[dt][v] = 0.f; }

    const int n_qtiles = (p.row_end - p.row_begin + BM - 1) / BM;
    const int n_iter = (kvb < kv_len) ? p.G * n_qtiles : 0;
    const float c = p.scale_log2e;
    constexpr float LOG2E = 1.4426950408889634f;

    // staging role of this thread: threads 0..127 carry Q, 128..255 carry dO
    const int st = tid & 127;
    const int s_chunk = st & 15, s_group = st >> 4;
    const bool is_do = tid >= 128;

    u32x4 pre[4];
    float pre_f = 0.f;   // tid < 32: LSE row, 32..63: delta row
    int pre_i = 0;       // 64..95: kv_start row, 96..127: kv_end row
    // token blocks of one kv head walk the (head, row tile) list from different
    // starting points so that their dQ atomics do not all hit the same rows
    const int it_shift = n_iter > 0 ? (int)(((int64_t)kblk * 7) % n_iter) : 0;
    auto prefetch = [&](int it0) {
        const int it = (it0 + it_shift) % n_iter;
        const int gi = it / n_qtiles, qt = it % n_qtiles;
        const int h = hk * p.G + gi;
        const int r0 = p.row_begin + qt * BM;
        const uint16_t* base = is_do ? p.dout + b * p.dos.b + h * p.dos.h
                                     : p.q + b * p.qs.b + h * p.qs.h;
        const int64_t rs = is_do ? p.dos.s : p.qs.s;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = r0 + 4 * s_group + i;
            pre[i] = ldg16(base + (int64_t)row * rs + s_chunk * 8, row < p.row_end);
        }
        if (tid < 64) {
            const int row = r0 + (tid & 31);
            const bool ok = row < p.row_end;
            const int64_t off = ((int64_t)b * p.Hq + h) * p.Lq + row;
            if (tid < 32) {
                const float l = ok ? p.lse[off] : -INFINITY;
                // exp2(x - inf) = 0: rows that saw no key (or do not exist) get P = 0
                pre_f = (l == -INFINITY) ? INFINITY : l * LOG2E;
            } else {
                pre_f = ok ? p.delta[off] : 0.f;
            }
        } else if (MASKED && tid < 128) {
            const int row = r0 + (tid & 31);
            const bool ok = row < p.row_end;
            const int64_t off = (int64_t)b * p.Lq + row;
            if (tid < 96) pre_i = ok ? p.kv_start[off] : 0;
            else pre_i = ok ? p.kv_end[off] : 0;
        }
    };

    if (n_iter > 0) prefetch(0);

    for (int it0 = 0; it0 < n_iter; ++it0) {
        const int it = (it0 + it_shift) % n_iter;
        const int gi = it / n_qtiles, qt = it % n_qtiles;
        const int h = hk * p.G + gi;
        const int r0 = p.row_begin + qt * BM;

        // ---- stage this step's Q / dO tile, row-major and transposed
        {
            uint16_t* rm = is_do ? dOs : Qs;
            uint16_t* tr = is_do ? dOT : QT;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                *reinterpret_cast<u32x4*>(&rm[(4 * s_group + i) * QS + s_chunk * 8]) = pre[i];
            u32x2 t8[8];
            transpose_4x8(pre, t8);
            const int pos = swap23(4 * s_group);
#pragma unroll
            for (int d = 0; d < 8; ++d)
                *reinterpret_cast<u32x2*>(&tr[(s_chunk * 8 + d) * TS + pos]) = t8[d];
            if (tid < 32) lse_s[tid] = pre_f;
            else if (tid < 64) delta_s[tid - 32] = pre_f;
            else if (MASKED && tid < 96) start_s[tid - 64] = pre_i;
            else if (MASKED && tid < 128) end_s[tid - 96] = pre_i;
        }
        __syncthreads();
        if (it0 + 1 < n_iter) prefetch(it0 + 1);

        // ---- S = Q K_w^T, dP = dO V_w^T : rows = text rows, cols = this wave's tokens
        f32x16 s, dp;
#pragma unroll
        for (int v = 0; v < 16; ++v) { s[v] = 0.f; dp[v] = 0.f; }
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            const bf16x8 aq = *reinterpret_cast<const bf16x8*>(&Qs[l32 * QS + kk * 16 + g * 8]);
            const bf16x8 ad = *reinterpret_cast<const bf16x8*>(&dOs[l32 * QS + kk * 16 + g * 8]);
            s = mfma32(aq, kreg[kk], s);
            dp = mfma32(ad, vreg[kk], dp);
        }

        // ---- P and dS (register v of lane-half g is text row 8*(v/4)+4g+(v%4))
#pragma unroll
        for (int vg = 0; vg < 4; ++vg) {
            const f32x4 l4 = *reinterpret_cast<const f32x4*>(&lse_s[8 * vg + 4 * g]);
            const f32x4 d4 = *reinterpret_cast<const f32x4*>(&delta_s[8 * vg + 4 * g]);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int v = 4 * vg + r;
                float pv = __builtin_amdgcn_exp2f(fmaf(s[v], c, -l4[r]));
                bool vis = kv_valid;
                if (MASKED) {
                    const int q_local = 8 * vg + 4 * g + r;
                    vis = vis && my_kv >= start_s[q_local] && my_kv < end_s[q_local];
                }
                pv = vis ? pv : 0.f;
                s[v] = pv;
                dp[v] = pv * (dp[v] - d4[r]);
            }
        }
        bf16x8 pb[2], dsb[2];
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

        // ---- dV_w^T += dO^T P,  dK_w^T += Q^T dS  (contraction over the 32 text rows)
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const bf16x8 a1 = *reinterpret_cast<const bf16x8*>(&dOT[(dt * 32 + l32) * TS + 16 * j + 8 * g]);
                const bf16x8 a2 = *reinterpret_cast<const bf16x8*>(&QT[(dt * 32 + l32) * TS + 16 * j + 8 * g]);
                dv[dt] = mfma32(a1, pb[j], dv[dt]);
                dk[dt] = mfma32(a2, dsb[j], dk[dt]);
            }

        // ---- hand dS to the other waves: dSs[text row][token of the block]
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int v = 8 * j + 2 * e;
                const uint32_t u = dsu[j][e];
#ifndef LVX_EXP_NO_DSWRITE
                dSs[acc_row(v, g) * DSS + 32 * wave + l32] = (uint16_t)(u & 0xffffu);
                dSs[acc_row(v + 1, g) * DSS + 32 * wave + l32] = (uint16_t)(u >> 16);
#endif
            }
        __syncthreads();

        // ---- dQ[rows, 32w..32w+31] = dS (A, from LDS) x K slice (B, registers).
        // A lane ends up with one head-dim column and 16 text rows, so every
        // atomic instruction covers two full 128-byte lines of dQ.
        f32x16 dq;
#pragma unroll
        for (int v = 0; v < 16; ++v) dq[v] = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const bf16x8 ao = *reinterpret_cast<const bf16x8*>(&dSs[l32 * DSS + 16 * j + 8 * g]);
            dq = mfma32(ao, ktreg[j], dq);
        }
        float* dqp = p.dq_acc + (((int64_t)b * p.Hq + h) * p.Lq + r0) * D + 32 * wave + l32;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int rl = acc_row(v, g);
#ifdef LVX_EXP_NO_ATOMICS
            if (dq[v] == 12345.678f) dqp[(int64_t)rl * D] = 1.f;
#else
            if (r0 + rl < p.row_end) unsafeAtomicAdd(dqp + (int64_t)rl * D, dq[v] * p.scale);
#endif
        }
        // no barrier here: the next step's staging writes only touch tiles every
        // wave finished reading before the barrier above, and dS is rewritten
        // only after the next step's first barrier
    }

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
                        a[r] += dk[dt][4 * vg + r] * p.scale;
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
                    a[0] = pack_bf16(dk[dt][4 * vg] * p.scale, dk[dt][4 * vg + 1] * p.scale);
                    a[1] = pack_bf16(dk[dt][4 * vg + 2] * p.scale, dk[dt][4 * vg + 3] * p.scale);
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
