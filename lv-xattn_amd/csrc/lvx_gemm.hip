// bf16 GEMM for the K/V recompute (K = X W_k, V = X W_v), its input gradient
// (dX = dK W_k^T + dV W_v^T, one GEMM whose contraction runs over two operand
// pairs) and the weight gradients (dW = X^T dK).  fp32 accumulate on
// v_mfma_f32_32x32x16_bf16, bf16 output.
//
// A work-group computes a 128 x 128 tile of C with 4 waves (64 x 64 each, 2 x 2
// MFMA tiles), stepping 64 along the contraction.  An operand whose memory has
// the contraction index contiguous is staged as [128][64+8] and read with
// 16-byte LDS reads; an operand whose memory has the OTHER index contiguous is
// staged exactly as it lies in memory, [64 k][128+32], and read with the
// transposing LDS read - nothing is transposed on the way in.  The MFMA
// computes C^T (A operand = rows of the B tile), so a lane ends up with 4
// consecutive columns of one C row and stores 8 bytes.
#include "lvx_common.hpp"
#include "lvx_kernels.hpp"

namespace lvx {

namespace {

constexpr int TM = 128, TN = 128, BK = 64;
constexpr int LS = BK + 8;     // row stride of a [row][k] tile (36 dwords)
constexpr int LT = TM + 32;    // row stride of a [k][row] tile (80 dwords)
constexpr int TILE_ELEMS = (TM * LS > BK * LT) ? TM * LS : BK * LT;

// Fetch the tile covering rows r0..r0+127 and k0..k0+63 into 4 x 16 bytes.
// ROW_CONTIG: memory is [k][row]; otherwise memory is [row][k].
template <bool ROW_CONTIG>
__device__ __forceinline__ void tile_load(u32x4 pre[4], const uint16_t* base, int64_t ld, int r0, int k0,
                                          int R, int K, int tid, int tiled_m = 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = tid + 256 * i;
        if (!ROW_CONTIG) {
            const int r = r0 + (c >> 3), k = k0 + (c & 7) * 8;
            pre[i] = ldg16(base + (int64_t)r * ld + k, r < R && k < K);
        } else {
            const int k = k0 + (c >> 4), r = r0 + (c & 15) * 8;
            const int64_t off = tiled_m ? ((int64_t)(k >> 7) * tiled_m + (r >> 5)) * 4096 + (k & 127) * 32 + (r & 31)
                                        : (int64_t)k * ld + r;
            pre[i] = ldg16(base + off, k < K && r < R);
        }
    }
}

template <bool ROW_CONTIG>
__device__ __forceinline__ void tile_store(const u32x4 pre[4], uint16_t* lds, int tid) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = tid + 256 * i;
        if (!ROW_CONTIG)
            *reinterpret_cast<u32x4*>(&lds[(c >> 3) * LS + (c & 7) * 8]) = pre[i];
        else
            *reinterpret_cast<u32x4*>(&lds[(c >> 4) * LT + (c & 15) * 8]) = pre[i];
    }
}

// MFMA operand for tile rows row0..row0+31 and k-step kk (16 values of k).
template <bool ROW_CONTIG>
__device__ __forceinline__ bf16x8 tile_operand(const uint16_t* lds, int row0, int kk, int lane, int tr_off) {
    if (!ROW_CONTIG)
        return *reinterpret_cast<const bf16x8*>(&lds[(row0 + (lane & 31)) * LS + kk * 16 + (lane >> 5) * 8]);
    return lds_operand_tr(&lds[tr_off + row0 + kk * 16 * LT], 4 * LT);
}

template <bool A_MCONTIG, bool B_NCONTIG>
__global__ __launch_bounds__(256, 2) void gemm_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(16))) uint16_t As[TILE_ELEMS];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[TILE_ELEMS];

    const int wid = xcd_remap(blockIdx.x, p.total_wg);
    if (wid >= p.total_wg) return;
    const int tn = wid % p.tiles_n;
    const int t1 = wid / p.tiles_n;
    const int tm = t1 % p.tiles_m;
    const int t2 = t1 / p.tiles_m;
    const int z = t2 % p.nbatch;
    const GemmProblem& pr = p.prob[t2 / p.nbatch];
    const int m0 = tm * TM, n0 = tn * TN;
    const int zo = z / p.batch_inner, zi = z % p.batch_inner;
    const int64_t a_off = (int64_t)z * p.a_batch;
    const int64_t b_off = zo * p.b_outer + (zi / p.b_group) * p.b_inner;
    uint16_t* const Cz = pr.C + zo * p.c_outer + zi * p.c_inner;
    int klen0 = pr.K[0];
    if (p.k_len) klen0 = min(klen0, p.k_len[zo]);

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int wm = wave & 1, wn = wave >> 1;
    const int tr_off = tr_lane_offset(lane, LT, false);

    f32x16 acc[2][2];   // [n tile][m tile]
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

    const int steps0 = (klen0 + BK - 1) / BK;
    const int steps1 = pr.nseg > 1 ? (pr.K[1] + BK - 1) / BK : 0;
    const int steps = steps0 + steps1;

    u32x4 apre[4], bpre[4];
    auto prefetch = [&](int s) {
        const int seg = s >= steps0 ? 1 : 0;
        const int k0 = (seg ? s - steps0 : s) * BK;
        const int kl = seg ? pr.K[1] : klen0;
        tile_load<A_MCONTIG>(apre, pr.A[seg] + a_off, pr.lda[seg], m0, k0, p.M_ld, kl, tid, p.a_tiled_m);
        tile_load<B_NCONTIG>(bpre, pr.Bm[seg] + b_off, pr.ldb[seg], n0, k0, p.N, kl, tid);
    };
    if (steps > 0) prefetch(0);

    for (int s = 0; s < steps; ++s) {
        __syncthreads();
        tile_store<A_MCONTIG>(apre, As, tid);
        tile_store<B_NCONTIG>(bpre, Bs, tid);
        __syncthreads();
        if (s + 1 < steps) prefetch(s + 1);
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            bf16x8 am[2], bn[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                am[t] = tile_operand<A_MCONTIG>(As, 64 * wm + 32 * t, kk, lane, tr_off);
                bn[t] = tile_operand<B_NCONTIG>(Bs, 64 * wn + 32 * t, kk, lane, tr_off);
            }
#pragma unroll
            for (int nt = 0; nt < 2; ++nt)
#pragma unroll
                for (int mt = 0; mt < 2; ++mt) acc[nt][mt] = mfma32(bn[nt], am[mt], acc[nt][mt]);
        }
    }

    // C^T tile: accumulator rows = n, cols = m
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
        const int m = m0 + 64 * wm + 32 * mt + l32;
        if (m >= p.M) continue;
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
            for (int vg = 0; vg < 4; ++vg) {
                const int n = n0 + 64 * wn + 32 * nt + 8 * vg + 4 * g;
                if (n < p.N) {
                    u32x2 w;
                    w[0] = pack_bf16(acc[nt][mt][4 * vg], acc[nt][mt][4 * vg + 1]);
                    w[1] = pack_bf16(acc[nt][mt][4 * vg + 2], acc[nt][mt][4 * vg + 3]);
                    *reinterpret_cast<u32x2*>(Cz + (int64_t)m * pr.ldc + n) = w;
                }
            }
    }
}

}  // namespace

hipError_t launch_gemm(const GemmParams& p, bool a_mcontig, bool b_ncontig, hipStream_t st) {
    const int grid = ((p.total_wg + 7) / 8) * 8;
    if (!a_mcontig && !b_ncontig)
        hipLaunchKernelGGL((gemm_kernel<false, false>), dim3(grid), dim3(256), 0, st, p);
    else if (!a_mcontig && b_ncontig)
        hipLaunchKernelGGL((gemm_kernel<false, true>), dim3(grid), dim3(256), 0, st, p);
    else if (a_mcontig && !b_ncontig)
        hipLaunchKernelGGL((gemm_kernel<true, false>), dim3(grid), dim3(256), 0, st, p);
    else
        hipLaunchKernelGGL((gemm_kernel<true, true>), dim3(grid), dim3(256), 0, st, p);
    return hipGetLastError();
}

}  // namespace lvx
