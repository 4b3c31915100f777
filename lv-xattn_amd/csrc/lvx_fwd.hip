// Flash cross-attention forward for gfx950: one launch computes, for a window
// of text rows, O = softmax(scale * Q K^T) V (bf16) and the per-row natural-log
// LSE against the local K/V shard (or one key split of it).
//
// Mapping.  A work-group is 4 wavefronts.  Each wavefront owns 32 text rows of
// ONE q head; the 4 waves of a group cover the q heads that share a kv head
// (G = 4: four heads x 32 rows; G = 1: one head x 128 rows), so the K/V tile
// staged in LDS is read by the whole GQA group and nothing is expanded in HBM.
//
// Per 64-key tile and wave (all MFMA are v_mfma_f32_32x32x16_bf16):
//   S^T[key, row]  = K_tile (A, from LDS)  x  Q^T (B, 32 VGPRs held for the whole kernel)
//   online softmax : a lane owns one text row (column of S^T) and 32 of the 64
//                    keys, so max/sum are in-register plus ONE exchange between
//                    the two lane halves; rescaling O is a per-lane scalar
//   O^T[d, row]   += V^T_tile (A, from LDS) x  P^T (B, straight from the S^T
//                    accumulators: register v of lane-half g is key
//                    8*(v/4)+4*g+(v%4); the V^T operand is fetched from the
//                    row-major V tile with the transposing LDS read, addressed
//                    in that same key order, so P never visits LDS and V is
//                    never transposed in memory)
// K and V are both staged row-major: K [64][128+8] (68-dword rows: the 16-byte
// operand reads of 16 consecutive lanes hit 64 distinct banks), V [64][128+16]
// (72-dword rows: the 8 rows x 16 dwords a transposing read touches tile the
// banks twice).  The LDS tiles are double-buffered: while tile t is consumed,
// tile t+1 moves from registers into the other buffer and tile t+2's global
// loads are issued, with one barrier per tile.  Loads past the end of the key
// range are clamped to its last row (those keys are masked out of S), so the
// loop body has no divergent branch.
#include "lvx_common.hpp"
#include "lvx_kernels.hpp"

namespace lvx {

namespace {

constexpr int D = 128;
constexpr int BN = 64;        // keys per tile
constexpr int KS = D + 8;     // K tile row stride (elements)
constexpr int VS = D + 16;    // V tile row stride (elements)
constexpr int BIG = 0x3fffffff;

template <bool MASKED>
__global__ __launch_bounds__(256, 2) void fwd_kernel(const FwdParams p) {
    __shared__ __attribute__((aligned(16))) uint16_t Ks2[2][BN * KS];
    __shared__ __attribute__((aligned(16))) uint16_t Vs2[2][BN * VS];
    __shared__ int red[4][4];

    const int wid = xcd_remap(blockIdx.x, p.total_wg);
    if (wid >= p.total_wg) return;
    const int tile = wid % p.n_row_tiles;
    const int t1 = wid / p.n_row_tiles;
    const int split = t1 % p.nsplit;
    const int t2 = t1 / p.nsplit;
    const int hg = t2 % p.n_head_groups;
    const int b = t2 / p.n_head_groups;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int h = hg * p.HG + (wave % p.HG);
    const int hk = h / p.G;
    const int row = p.row_begin + (tile * p.RS + wave / p.HG) * 32 + l32;
    const bool row_ok = row < p.row_end;

    int kv_len = p.Lkv;
    if (p.kv_len) kv_len = min(p.kv_len[b], p.Lkv);
    const int kv_lo = split * p.split_len;
    const int kv_hi = min(kv_len, kv_lo + p.split_len);

    // this lane's visible key interval
    int my_s = kv_lo, my_e = kv_hi;
    if (MASKED) {
        if (row_ok) {
            my_s = max(kv_lo, p.kv_start[(int64_t)b * p.Lq + row]);
            my_e = min(kv_hi, p.kv_end[(int64_t)b * p.Lq + row]);
        } else {
            my_e = my_s;
        }
    }
    if (my_e <= my_s) { my_s = BIG; my_e = 0; }

    // work-group key range: [lo, hi) covers every non-empty row; tiles inside
    // [in_lo, in_hi) are visible to every row and need no masking
    int lo = my_s, hi = my_e, in_lo = my_s, in_hi = my_e;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        lo = min(lo, __shfl_xor(lo, off));
        hi = max(hi, __shfl_xor(hi, off));
        in_lo = max(in_lo, __shfl_xor(in_lo, off));
        in_hi = min(in_hi, __shfl_xor(in_hi, off));
    }
    if (lane == 0) { red[wave][0] = lo; red[wave][1] = hi; red[wave][2] = in_lo; red[wave][3] = in_hi; }
    __syncthreads();
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        lo = min(lo, red[w][0]);
        hi = max(hi, red[w][1]);
        in_lo = max(in_lo, red[w][2]);
        in_hi = min(in_hi, red[w][3]);
    }

    // Q^T as B operand, resident for the whole kernel
    bf16x8 qreg[8];
    {
        const uint16_t* qp = p.q + b * p.qs.b + h * p.qs.h + (int64_t)row * p.qs.s + g * 8;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) qreg[kk] = as_bf16x8(ldg16(qp + kk * 16, row_ok));
    }

    const uint16_t* kbase = p.k + b * p.ks.b + hk * p.ks.h;
    const uint16_t* vbase = p.v + b * p.vs.b + hk * p.vs.h;
    const int off_vT = tr_lane_offset(lane, VS, true);   // V^T operand, keys in accumulator order

    u32x4 kpre[4], vpre[4];
    const int ld_row = tid >> 4, ld_col = (tid & 15) * 8;   // this thread's chunk of rows ld_row + 16 i
    auto prefetch = [&](int kv0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int kv = min(kv0 + ld_row + 16 * i, kv_hi - 1);
            kpre[i] = *reinterpret_cast<const u32x4*>(kbase + (int64_t)kv * p.ks.s + ld_col);
            vpre[i] = *reinterpret_cast<const u32x4*>(vbase + (int64_t)kv * p.vs.s + ld_col);
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<u32x4*>(&Ks2[buf][(ld_row + 16 * i) * KS + ld_col]) = kpre[i];
            *reinterpret_cast<u32x4*>(&Vs2[buf][(ld_row + 16 * i) * VS + ld_col]) = vpre[i];
        }
    };

    f32x16 acc[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[dt][v] = 0.f;
    float m_i = -INFINITY, l_i = 0.f;
    const float c = p.scale_log2e;

    const int t_begin = (hi > lo) ? lo / BN : 0;
    const int t_end = (hi > lo) ? (hi + BN - 1) / BN : 0;
    if (t_end > t_begin) {
        prefetch(t_begin * BN);
        stage(0);
        __syncthreads();
        prefetch(min(t_begin + 1, t_end - 1) * BN);
    }

    for (int t = t_begin; t < t_end; ++t) {
        const int kv0 = t * BN;
        const int buf = (t - t_begin) & 1;
        const uint16_t* Ks = Ks2[buf];
        const uint16_t* Vs = Vs2[buf];

        // S^T = K Q^T : rows = keys (two 32-key sub-tiles), cols = text rows
        f32x16 s0, s1;
#pragma unroll
        for (int v = 0; v < 16; ++v) { s0[v] = 0.f; s1[v] = 0.f; }
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            const bf16x8 a0 = *reinterpret_cast<const bf16x8*>(&Ks[l32 * KS + kk * 16 + g * 8]);
            const bf16x8 a1 = *reinterpret_cast<const bf16x8*>(&Ks[(32 + l32) * KS + kk * 16 + g * 8]);
            s0 = mfma32(a0, qreg[kk], s0);
            s1 = mfma32(a1, qreg[kk], s1);
        }

        if (kv0 < in_lo || kv0 + BN > in_hi) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int kv = kv0 + acc_row(v, g);
                if (kv < my_s || kv >= my_e) s0[v] = -INFINITY;
                if (kv + 32 < my_s || kv + 32 >= my_e) s1[v] = -INFINITY;
            }
        }

        float mx = fmaxf(s0[0], s1[0]);
#pragma unroll
        for (int v = 1; v < 16; ++v) mx = fmaxf(mx, fmaxf(s0[v], s1[v]));
        {   // other half of the wave holds the other 32 keys of the same text row
            const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
            mx = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
        }
        const float m_new = fmaxf(m_i, mx);
        const float mc = (m_new == -INFINITY) ? 0.f : m_new * c;
        const float alpha = __builtin_amdgcn_exp2f(m_i * c - mc);
        m_i = m_new;

        float rs = 0.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            s0[v] = __builtin_amdgcn_exp2f(fmaf(s0[v], c, -mc));
            s1[v] = __builtin_amdgcn_exp2f(fmaf(s1[v], c, -mc));
            rs += s0[v] + s1[v];
        }
        l_i = l_i * alpha + rs;

        // P^T as B operand: k-step j covers keys 16j..16j+15 of the tile
        bf16x8 pb[4];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            u32x4 u0, u1;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                u0[e] = pack_bf16(s0[8 * j + 2 * e], s0[8 * j + 2 * e + 1]);
                u1[e] = pack_bf16(s1[8 * j + 2 * e], s1[8 * j + 2 * e + 1]);
            }
            pb[j] = as_bf16x8(u0);
            pb[2 + j] = as_bf16x8(u1);
        }

        if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {   // the running max moved for some row
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[dt][v] *= alpha;
        }

        // O^T += V^T P^T
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bf16x8 a = lds_operand_tr(&Vs[off_vT + 16 * j * VS + dt * 32], 8 * VS);
                acc[dt] = mfma32(a, pb[j], acc[dt]);
            }

        // tile t+1 (in registers since the previous iteration) goes to the other
        // buffer, whose last readers finished before the previous barrier
        if (t + 1 < t_end) {
            stage(buf ^ 1);
            __syncthreads();
            prefetch(min(t + 2, t_end - 1) * BN);
        }
    }

    // epilogue: the two lane halves hold partial row sums of the same row
    const float l_tot = l_i + __shfl_xor(l_i, 32);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (row_ok) {
        uint16_t* op = p.o + split * p.o_split_stride + b * p.os.b + h * p.os.h + (int64_t)row * p.os.s;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int vg = 0; vg < 4; ++vg) {
                u32x2 w;
                w[0] = pack_bf16(acc[dt][4 * vg] * inv, acc[dt][4 * vg + 1] * inv);
                w[1] = pack_bf16(acc[dt][4 * vg + 2] * inv, acc[dt][4 * vg + 3] * inv);
                *reinterpret_cast<u32x2*>(op + dt * 32 + 8 * vg + 4 * g) = w;
            }
        if (g == 0) {
            const float lse = l_tot > 0.f ? m_i * p.scale + __logf(l_tot) : -INFINITY;
            p.lse[split * p.lse_split_stride + ((int64_t)b * p.Hq + h) * p.lse_bh_stride + row] = lse;
        }
    }
}

}  // namespace

hipError_t launch_fwd(const FwdParams& p, bool masked, hipStream_t st) {
    const int grid = ((p.total_wg + 7) / 8) * 8;
    if (masked)
        hipLaunchKernelGGL(fwd_kernel<true>, dim3(grid), dim3(256), 0, st, p);
    else
        hipLaunchKernelGGL(fwd_kernel<false>, dim3(grid), dim3(256), 0, st, p);
    return hipGetLastError();
}

}  // namespace lvx
