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
// Per 32-row step and wave (all MFMA are 32x32x16 bf16):
//   S, dP        2 x 8 MFMA   A = Q / dO rows from LDS (16-byte reads)
//   dV^T, dK^T   2 x 8 MFMA   A = dO^T / Q^T, read from the SAME row-major LDS
//                             tiles with the transposing LDS read; B = P / dS
//                             straight from the accumulators (the transposing
//                             read is addressed in the accumulator's row order)
//   dQ           8 MFMA       A = dS, read transposed from the dS^T tile the
//                             waves wrote (8-byte writes), B = K slice
#include "lvx_common.hpp"
#include "lvx_kernels.hpp"

namespace lvx {

namespace {

constexpr int D = 128;
constexpr int BN = 128;       // visual tokens per work-group
constexpr int BM = 32;        // text rows per step
constexpr int QS = D + 8;     // row stride of the Q / dO tiles (68 dwords: 16-byte row reads conflict-free)
constexpr int DSS = BM + 4;   // row stride of the dS^T tile [token][row] (18 dwords)
constexpr int KPS = D + 8;    // row stride of the K tile staged once in the prologue

constexpr int OFF_Q = 0;
constexpr int OFF_DO = OFF_Q + BM * QS;
constexpr int OFF_DS = OFF_DO + BM * QS;
constexpr int LOOP_ELEMS = OFF_DS + BN * DSS;
constexpr int PRO_ELEMS = BN * KPS;
constexpr int SMEM_ELEMS = LOOP_ELEMS > PRO_ELEMS ? LOOP_ELEMS : PRO_ELEMS;

template <bool MASKED>
__global__ __launch_bounds__(256, 1) void bwd_kernel(const BwdParams p) {
    __shared__ __attribute__((aligned(16))) uint16_t smem[SMEM_ELEMS];
    // per-row metadata of the staged tile: [0,32) LSE*log2e, [32,64) delta,
    // [64,96) kv_start, [96,128) kv_end (raw 32-bit words)
    __shared__ u32x4 meta_s4[BM];
    uint32_t* meta_s = reinterpret_cast<uint32_t*>(meta_s4);
    const u32x4* lse_s4 = meta_s4;            // 8 x 16 bytes each
    const u32x4* delta_s4 = meta_s4 + 8;
    const u32x4* start_s4 = meta_s4 + 16;
    const u32x4* end_s4 = meta_s4 + 24;

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

    uint16_t* Qs = smem + OFF_Q;
    uint16_t* dOs = smem + OFF_DO;
    uint16_t* dST = smem + OFF_DS;

    const uint16_t* kbase = p.k + b * p.ks.b + hk * p.ks.h;
    const uint16_t* vbase = p.v + b * p.vs.b + hk * p.vs.h;

    // ---- prologue: K, V rows of this wave as B operands (contraction over d),
    //      and the K slice [tokens of the block][32w..32w+31] as B operand for dQ
    //      (contraction over the tokens)
    bf16x8 kreg[8], vreg[8], ktreg[8];
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
        kreg[kk] = as_bf16x8(ldg16(kbase + (int64_t)my_kv * p.ks.s + kk * 16 + g * 8, kv_valid));
        vreg[kk] = as_bf16x8(ldg16(vbase + (int64_t)my_kv * p.vs.s + kk * 16 + g * 8, kv_valid));
    }
    {
        uint16_t* Kp = smem;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int c = tid + 256 * i;
            const int kv = kvb + (c >> 4);
            *reinterpret_cast<u32x4*>(&Kp[(c >> 4) * KPS + (c & 15) * 8]) =
                ldg16(kbase + (int64_t)kv * p.ks.s + (c & 15) * 8, kv < kv_len);
        }
        __syncthreads();
        const int off = tr_lane_offset(lane, KPS, false) + 32 * wave;
#pragma unroll
        for (int j = 0; j < 8; ++j) ktreg[j] = lds_operand_tr(&Kp[off + 16 * j * KPS], 4 * KPS);
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
    uint16_t* stage_dst = (is_do ? dOs : Qs) + 4 * s_group * QS + s_chunk * 8;

    const int dq_lane = 4 * g * D + 32 * wave + l32;   // this lane's element offset inside a dQ tile

    // per-lane offsets of the transposing operand reads
    const int off_qT = tr_lane_offset(lane, QS, true);     // Q^T / dO^T, rows in accumulator order
    const int off_dsT = tr_lane_offset(lane, DSS, false);  // dS from dS^T, tokens in natural order

    u32x4 pre[4];
    uint32_t pre_m = 0;
    // Every load below is unconditional: rows past the window are clamped to its
    // last row (their LSE is forced to +inf, so P = 0 and nothing they carry
    // reaches a result), and the step after the last one re-reads the last.
    const int meta_kind = (tid >> 5) & 3;    // 0 LSE, 1 delta, 2 kv_start, 3 kv_end
    // token blocks of one kv head walk the (head, row tile) list from different
    // starting points so that their dQ atomics do not all hit the same rows
    const int it_shift = n_iter > 0 ? (int)(((int64_t)kblk * 7) % n_iter) : 0;
    auto prefetch = [&](int it0) {
        const int it = (min(it0, n_iter - 1) + it_shift) % n_iter;
        const int gi = it / n_qtiles, qt = it % n_qtiles;
        const int h = hk * p.G + gi;
        const int r0 = p.row_begin + qt * BM;
        const uint16_t* base = is_do ? p.dout + b * p.dos.b + h * p.dos.h
                                     : p.q + b * p.qs.b + h * p.qs.h;
        const int64_t rs = is_do ? p.dos.s : p.qs.s;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = min(r0 + 4 * s_group + i, p.row_end - 1);
            pre[i] = *reinterpret_cast<const u32x4*>(base + (int64_t)row * rs + s_chunk * 8);
        }
        const int mrow = r0 + (tid & 31);
        const bool ok = mrow < p.row_end;
        const int crow = min(mrow, p.row_end - 1);
        const int64_t off_bh = ((int64_t)b * p.Hq + h) * p.Lq + crow;
        const int64_t off_b = (int64_t)b * p.Lq + crow;
        const uint32_t* src = reinterpret_cast<const uint32_t*>(p.lse) + off_bh;
        if (meta_kind == 1) src = reinterpret_cast<const uint32_t*>(p.delta) + off_bh;
        if (MASKED && meta_kind == 2) src = reinterpret_cast<const uint32_t*>(p.kv_start) + off_b;
        if (MASKED && meta_kind == 3) src = reinterpret_cast<const uint32_t*>(p.kv_end) + off_b;
        const uint32_t raw = *src;
        const float l = __uint_as_float(raw);
        // exp2(x - inf) = 0: rows that saw no key (or do not exist) get P = 0
        const float lt = (!ok || l == -INFINITY) ? INFINITY : l * LOG2E;
        pre_m = meta_kind == 0 ? __float_as_uint(lt) : (ok ? raw : 0u);
    };

    if (n_iter > 0) prefetch(0);

    for (int it0 = 0; it0 < n_iter; ++it0) {
        const int it = (it0 + it_shift) % n_iter;
        const int gi = it / n_qtiles, qt = it % n_qtiles;
        const int h = hk * p.G + gi;
        const int r0 = p.row_begin + qt * BM;

        // ---- stage this step's Q / dO tile (row-major only)
#pragma unroll
        for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(stage_dst + i * QS) = pre[i];
        meta_s[tid & 127] = pre_m;     // both halves of the group write the same words
        __syncthreads();
        prefetch(it0 + 1);

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

        // ---- P and scale*dS (register v of lane-half g is text row 8*(v/4)+4g+(v%4))
#pragma unroll
        for (int vg = 0; vg < 4; ++vg) {
            const f32x4 l4 = __builtin_bit_cast(f32x4, lse_s4[2 * vg + g]);
            const f32x4 d4 = __builtin_bit_cast(f32x4, delta_s4[2 * vg + g]);
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
                const u32x4 sp = start_s4[2 * vg + g];
                const u32x4 ep = end_s4[2 * vg + g];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const bool vis = kv_valid && my_kv >= (int)sp[r] && my_kv < (int)ep[r];
                    s[4 * vg + r] = vis ? s[4 * vg + r] : 0.f;
                    dp[4 * vg + r] = vis ? dp[4 * vg + r] : 0.f;
                }
            }
        } else if (tail_block) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                s[v] = kv_valid ? s[v] : 0.f;
                dp[v] = kv_valid ? dp[v] : 0.f;
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

        // ---- hand scale*dS to the other waves: dST[token of the block][text row]
        {
            uint16_t* dsp = &dST[(32 * wave + l32) * DSS + 4 * g];
#pragma unroll
            for (int vg = 0; vg < 4; ++vg) {
                const u32x2 w = {dsu[vg >> 1][2 * (vg & 1)], dsu[vg >> 1][2 * (vg & 1) + 1]};
                *reinterpret_cast<u32x2*>(dsp + 8 * vg) = w;
            }
        }

        // ---- dV_w^T += dO^T P,  dK_w^T += Q^T (scale*dS)  (contraction over the 32 text rows)
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const bf16x8 a1 = lds_operand_tr(&dOs[off_qT + 16 * j * QS + dt * 32], 8 * QS);
                const bf16x8 a2 = lds_operand_tr(&Qs[off_qT + 16 * j * QS + dt * 32], 8 * QS);
                dv[dt] = mfma32(a1, pb[j], dv[dt]);
                dk[dt] = mfma32(a2, dsb[j], dk[dt]);
            }
        __syncthreads();

        // ---- dQ[rows, 32w..32w+31] = (scale*dS) (A, transposed read) x K slice (B, registers).
        // A lane ends up with one head-dim column and 16 text rows, so every
        // atomic instruction covers two full 128-byte lines of dQ.
        f32x16 dq;
#pragma unroll
        for (int v = 0; v < 16; ++v) dq[v] = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const bf16x8 ao = lds_operand_tr(&dST[off_dsT + 16 * j * DSS], 4 * DSS);
            dq = mfma32(ao, ktreg[j], dq);
        }
        float* dqp = p.dq_acc + (((int64_t)b * p.Hq + h) * p.Lq + r0) * D;   // uniform
        if (r0 + BM <= p.row_end) {
#pragma unroll
            for (int v = 0; v < 16; ++v) unsafeAtomicAdd(dqp + (dq_lane + (8 * (v >> 2) + (v & 3)) * D), dq[v]);
        } else {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int rl = acc_row(v, g);
                if (r0 + rl < p.row_end) unsafeAtomicAdd(dqp + (dq_lane + (8 * (v >> 2) + (v & 3)) * D), dq[v]);
            }
        }
        // no barrier here: the next step's staging writes only touch tiles every
        // wave finished reading before the barrier above, and dS^T is rewritten
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
