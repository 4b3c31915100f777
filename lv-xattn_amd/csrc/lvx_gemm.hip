// bf16 GEMM for the K/V recompute (K = X W_k, V = X W_v), its input gradient
// (dX = dK W_k^T + dV W_v^T, one GEMM whose contraction runs over two operand
// pairs) and the weight gradients (dW = X^T dK).  fp32 accumulate on
// v_mfma_f32_32x32x16_bf16, bf16 output.
//
// A work-group computes a (64 WM) x (64 WN) tile of C with 4 waves in a 2 x 2
// grid, each wave WM x WN MFMA tiles, stepping 64 along the contraction.  The
// default is 256 x 128 (wave tile 128 x 64): every LDS operand read then feeds
// 2 or 4 MFMAs, which keeps the LDS pipe well below the MFMA pipe.  An operand
// whose memory has the contraction index contiguous is staged as [rows][64+8]
// and read with 16-byte LDS reads; an operand whose memory has the OTHER index
// contiguous is staged exactly as it lies in memory, [64 k][rows+32], and read
// with the transposing LDS read - nothing is transposed on the way in.  The
// MFMA computes C^T (A operand = rows of the B tile), so a lane ends up with 4
// consecutive columns of one C row and stores 8 bytes.
#include "lvx_common.hpp"
#include "lvx_kernels.hpp"

namespace lvx {

namespace {

constexpr int BK = 64;
constexpr int LS = BK + 8;     // row stride of a [row][k] tile (36 dwords)
// a tile of ROWS rows: [ROWS][LS] or [BK][ROWS + 32] (row stride = 16 mod 64 dwords)
constexpr int tile_elems(int rows) { return rows * LS > BK * (rows + 32) ? rows * LS : BK * (rows + 32); }

// Global -> LDS staging of one operand tile (ROWS rows x 64 k), ROWS/32 chunks of
// 16 bytes per thread.  ROW_CONTIG: memory is [k][row]; otherwise [row][k].
// Every load is `uniform stage base + per-thread 32-bit byte offset`: the
// offsets are computed once (rows past the end are clamped onto a valid row;
// their products are never stored), the base advances by one k-step per
// stage, so the steady-state loop issues bare loads with no address arithmetic.
// Only the last stage of a contraction segment, when it is partial, re-derives
// clamped offsets and zeroes the chunks whose k lies past the end.
template <bool ROW_CONTIG, int ROWS>
struct TileLoader {
    static constexpr int NCH = ROWS / 32;
    static constexpr int CPR = ROWS / 8;      // chunks per k row of a [k][row] tile
    static constexpr int LT = ROWS + 32;
    uint32_t voff[NCH];
    u32x4 pre[NCH];
    uint32_t kstep_bytes;                      // byte distance of one k row (ROW_CONTIG) or 2

    __device__ __forceinline__ static int kpos(int c) { return ROW_CONTIG ? c / CPR : (c & 7) * 8; }

    __device__ __forceinline__ void setup(int64_t ld, int r0, int R, int tid, int tiled_m) {
        kstep_bytes = ROW_CONTIG ? (tiled_m ? 64u : (uint32_t)ld * 2u) : 2u;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + 256 * i;
            if (!ROW_CONTIG) {
                const int r = min(r0 + (c >> 3), R - 1) - r0;
                voff[i] = (uint32_t)r * (uint32_t)ld * 2u + (uint32_t)(c & 7) * 16u;
            } else if (tiled_m) {
                const int r = min(r0 + (c % CPR) * 8, R - 8);
                voff[i] = (uint32_t)((c / CPR) * 32 + (r >> 5) * 4096 + (r & 31)) * 2u;
            } else {
                const int r = min(r0 + (c % CPR) * 8, R - 8) - r0;
                voff[i] = (uint32_t)(c / CPR) * (uint32_t)ld * 2u + (uint32_t)r * 2u;
            }
        }
    }

    // base: address of (row r0, k0) of the operand (tiled: of the k0 tile row); krem = K - k0 > 0
    __device__ __forceinline__ void load(const char* base, int krem, int tid) {
        if (krem >= BK) {
#pragma unroll
            for (int i = 0; i < NCH; ++i) pre[i] = *reinterpret_cast<const u32x4*>(base + voff[i]);
        } else {
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const int kp = kpos(tid + 256 * i);
                const uint32_t back = (uint32_t)kp * kstep_bytes;
                pre[i] = *reinterpret_cast<const u32x4*>(base + (kp < krem ? voff[i] : voff[i] - back));
            }
        }
    }

    __device__ __forceinline__ void store(uint16_t* lds, int krem, int tid) {
        if (krem < BK) {
            const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int i = 0; i < NCH; ++i)
                if (kpos(tid + 256 * i) >= krem) pre[i] = z;
        }
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + 256 * i;
            if (!ROW_CONTIG)
                *reinterpret_cast<u32x4*>(&lds[(c >> 3) * LS + (c & 7) * 8]) = pre[i];
            else
                *reinterpret_cast<u32x4*>(&lds[(c / CPR) * LT + (c % CPR) * 8]) = pre[i];
        }
    }
};

// MFMA operand for tile rows row0..row0+31 and k-step kk (16 values of k).
template <bool ROW_CONTIG, int ROWS>
__device__ __forceinline__ bf16x8 tile_operand(const uint16_t* lds, int row0, int kk, int lane, int tr_off) {
    constexpr int LT = ROWS + 32;
    if (!ROW_CONTIG)
        return *reinterpret_cast<const bf16x8*>(&lds[(row0 + (lane & 31)) * LS + kk * 16 + (lane >> 5) * 8]);
    return lds_operand_tr(&lds[tr_off + row0 + kk * 16 * LT], 4 * LT);
}

template <bool A_MCONTIG, bool B_NCONTIG, int WM, int WN>
__global__ __launch_bounds__(256, 2) void gemm_kernel(const GemmParams p) {
    constexpr int TM = 64 * WM, TN = 64 * WN;
    __shared__ __attribute__((aligned(16))) uint16_t As[tile_elems(TM)];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[tile_elems(TN)];

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
    const int tr_off_a = tr_lane_offset(lane, TM + 32, false);
    const int tr_off_b = tr_lane_offset(lane, TN + 32, false);

    f32x16 acc[WN][WM];   // [n tile][m tile]
#pragma unroll
    for (int a = 0; a < WN; ++a)
#pragma unroll
        for (int b = 0; b < WM; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

    const int steps0 = (klen0 + BK - 1) / BK;
    const int steps1 = pr.nseg > 1 ? (pr.K[1] + BK - 1) / BK : 0;
    const int steps = steps0 + steps1;

    TileLoader<A_MCONTIG, TM> la;
    TileLoader<B_NCONTIG, TN> lb;
    const char* abase = nullptr;
    const char* bbase = nullptr;
    int64_t a_kstride = 0, b_kstride = 0;   // bytes per 64 k
    int seg_len = 0, seg_first = 0;
    auto enter_segment = [&](int seg) {
        const int64_t lda = pr.lda[seg], ldb = pr.ldb[seg];
        la.setup(lda, m0, p.M_ld, tid, p.a_tiled_m);
        lb.setup(ldb, n0, p.N, tid, 0);
        abase = reinterpret_cast<const char*>(pr.A[seg] + a_off);
        if (!p.a_tiled_m) abase += (A_MCONTIG ? (int64_t)m0 : (int64_t)m0 * lda) * 2;
        bbase = reinterpret_cast<const char*>(pr.Bm[seg] + b_off) + (B_NCONTIG ? (int64_t)n0 : (int64_t)n0 * ldb) * 2;
        a_kstride = A_MCONTIG ? (p.a_tiled_m ? 0 : lda * BK * 2) : BK * 2;
        b_kstride = B_NCONTIG ? ldb * BK * 2 : BK * 2;
        seg_len = seg ? pr.K[1] : klen0;
        seg_first = seg ? steps0 : 0;
    };
    // issue the loads of stage s; returns K - k0 of that stage
    auto prefetch = [&](int s) {
        if (s == 0 && steps0 > 0) enter_segment(0);
        else if (s == steps0) enter_segment(1);
        const int ks = s - seg_first;
        const int krem = seg_len - ks * BK;
        const char* ab = abase + ks * a_kstride;
        if (A_MCONTIG && p.a_tiled_m)   // tile row of 128 k: [k / 128][m / 32][128][32]
            ab = abase + ((int64_t)(ks >> 1) * p.a_tiled_m * 4096 + (ks & 1) * 2048) * 2;
        la.load(ab, krem, tid);
        lb.load(bbase + ks * b_kstride, krem, tid);
        return krem;
    };
    int krem = BK;
    if (steps > 0) krem = prefetch(0);

    for (int s = 0; s < steps; ++s) {
        __syncthreads();
        la.store(As, krem, tid);
        lb.store(Bs, krem, tid);
        __syncthreads();
        if (s + 1 < steps) krem = prefetch(s + 1);
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            bf16x8 am[WM], bn[WN];
#pragma unroll
            for (int t = 0; t < WM; ++t) am[t] = tile_operand<A_MCONTIG, TM>(As, 32 * (WM * wm + t), kk, lane, tr_off_a);
#pragma unroll
            for (int t = 0; t < WN; ++t) bn[t] = tile_operand<B_NCONTIG, TN>(Bs, 32 * (WN * wn + t), kk, lane, tr_off_b);
#pragma unroll
            for (int nt = 0; nt < WN; ++nt)
#pragma unroll
                for (int mt = 0; mt < WM; ++mt) acc[nt][mt] = mfma32(bn[nt], am[mt], acc[nt][mt]);
        }
    }

    // C^T tile: accumulator rows = n, cols = m
#pragma unroll
    for (int mt = 0; mt < WM; ++mt) {
        const int m = m0 + 32 * (WM * wm + mt) + l32;
        if (m >= p.M) continue;
#pragma unroll
        for (int nt = 0; nt < WN; ++nt)
#pragma unroll
            for (int vg = 0; vg < 4; ++vg) {
                const int n = n0 + 32 * (WN * wn + nt) + 8 * vg + 4 * g;
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
        hipLaunchKernelGGL((gemm_kernel<false, false, GEMM_WM, GEMM_WN>), dim3(grid), dim3(256), 0, st, p);
    else if (!a_mcontig && b_ncontig)
        hipLaunchKernelGGL((gemm_kernel<false, true, GEMM_WM, GEMM_WN>), dim3(grid), dim3(256), 0, st, p);
    else if (a_mcontig && !b_ncontig)
        hipLaunchKernelGGL((gemm_kernel<true, false, GEMM_WM, GEMM_WN>), dim3(grid), dim3(256), 0, st, p);
    else
        hipLaunchKernelGGL((gemm_kernel<true, true, GEMM_WM, GEMM_WN>), dim3(grid), dim3(256), 0, st, p);
    return hipGetLastError();
}

}  // namespace lvx
