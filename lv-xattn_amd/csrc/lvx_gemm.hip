// bf16 GEMM for the K/V recompute (K = X W_k, V = X W_v), its input gradient
// (dX = dK W_k^T + dV W_v^T, one GEMM whose contraction runs over two operand
// pairs), the weight gradients (dW = X^T dK) and the batched dQ = dS K of the
// attention backward.  fp32 accumulate on v_mfma_f32_32x32x16_bf16, bf16 output.
//
// Structure (8 waves, two per SIMD, in lock-step "ping-pong"):
//  * Operand tiles go from global memory straight into LDS with
//    global_load_lds_dwordx4 (no staging registers), NS stages of 32 k deep, so
//    a tile is requested NS-1 stages before it is used.
//  * Waves 0-3 and waves 4-7 (one of each per SIMD) run the same loop half a
//    stage apart: while one set issues the 16 MFMAs of a stage from registers,
//    the other set fetches its operands of the next stage from LDS and issues
//    its share of the global loads; a work-group barrier after every phase
//    keeps the two sets alternating, so the MFMA pipe of every SIMD always has
//    one wave feeding it and the LDS / memory latency of the other is hidden.
//  * The direct-to-LDS load writes 64 lanes x 16 bytes contiguously, so tiles
//    cannot be padded; bank conflicts are avoided by permuting 16-byte chunks
//    (an XOR of the chunk index with row bits), applied on the global-address
//    side when loading and on the LDS-address side when reading.
//  * An operand whose memory has the contraction index contiguous is read
//    with 16-byte LDS reads; one whose memory has the OTHER index contiguous
//    is kept as it lies, [k][rows], and read with the transposing LDS read.
//  * The MFMA computes C^T (A operand = rows of the B tile), so a lane ends up
//    with 4 consecutive columns of one C row and stores 8 bytes.
#include <type_traits>

#include "lvx_common.hpp"
#include "lvx_kernels.hpp"

namespace lvx {

namespace {

// registers the hand-scheduled loop uses besides its operands (see gen_gemm_loop.py)
#define LVX_GEMM_LOOP_CLOBBERS "v128", "v129", "v130", "v131", "v132", "v133", "v134", "v135", "v136", "v137", "v138", "v139", "v140", "v141", "v142", "v143", "v144", "v145", "v146", "v147", "v148", "v149", "v150", "v151", "v152", "v153", "v154", "v155", "v156", "v157", "v158", "v159", "v160", "v161", "v162", "v163", "v164", "v165", "v166", "v167", "v168", "v169", "v170", "v171", "v172", "v173", "v174", "v175", "v176", "v177", "v178", "v179", "v180", "v181", "v182", "v183", "v184", "v185", "v186", "v187", "v188", "v189", "v190", "v191", "v192", "v193", "v194", "v195", "v196", "v197", "v198", "v199", "v200", "v201", "v202", "v203", "v204", "v205", "v206", "v207", "v208", "v209", "v210", "v211", "v212", "v213", "v214", "v215", "v216", "v217", "v218", "v219", "v220", "v221", "v222", "v223"

constexpr int BK = 32;                 // contraction depth of one stage
__device__ uint32_t zero_chunk[4];     // source of the chunks past the end of a contraction

__device__ __forceinline__ void phase_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
}

// One operand's part of a stage: ROWS rows x 32 k, unpadded, in wave-chunks of
// 1 KiB (what one global_load_lds_dwordx4 writes).
//   !ROW_CONTIG (memory [row][k]): LDS row r at r*64 B; its 16-byte chunk c
//       (k = 8c..8c+7) sits at position c ^ ((r >> 2) & 3).
//    ROW_CONTIG (memory [k][row]): LDS k-row at k*ROWS*2 B; its chunk q (rows
//       8q..8q+7) sits at position q ^ ((k & 3) << 2).
template <bool ROW_CONTIG, int ROWS>
struct Region {
    static constexpr int BYTES = ROWS * BK * 2;
    static constexpr int CHUNKS = BYTES / 1024;
    static constexpr int LPR = ROWS / 8;          // lanes per k-row (ROW_CONTIG)

    // what lane `lane` of the wave loading chunk `ch` fetches: byte offset from the
    // stage base of the operand, and the k position inside the stage
    __device__ __forceinline__ static uint32_t src(int ch, int lane, int r0, int R, int64_t ld, int tiled_m,
                                                   int& kpos) {
        if (!ROW_CONTIG) {
            const int row = 16 * ch + (lane >> 2);
            const int c = (lane & 3) ^ ((lane >> 4) & 3);
            kpos = c * 8;
            return (uint32_t)(min(r0 + row, R - 1) - r0) * (uint32_t)ld * 2u + (uint32_t)c * 16u;
        }
        const int k = ch * (64 / LPR) + lane / LPR;
        const int q = (lane % LPR) ^ ((k & 3) << 2);
        kpos = k;
        const int r = min(r0 + q * 8, R - 8);
        if (tiled_m) return (uint32_t)(k * 32 + (r >> 5) * 4096 + (r & 31)) * 2u;
        return (uint32_t)k * (uint32_t)ld * 2u + (uint32_t)(r - r0) * 2u;
    }

    // per-lane LDS byte offsets for the operand reads of a wave whose first
    // 32-row tile in the region is tile j0 (W tiles per wave).
    //  !ROW_CONTIG: rd[kk] for k-step kk; add tile * 2048
    //   ROW_CONTIG: rd[t] for tile t; add kk * 16 * ROWS * 2 (+ 4 * ROWS * 2 for the second half)
    template <int W>
    __device__ __forceinline__ static void read_offsets(uint32_t* rd, int j0, int lane) {
        if (!ROW_CONTIG) {
            const int l32 = lane & 31, g = lane >> 5, s = (l32 >> 2) & 3;
            rd[0] = (uint32_t)(j0 * 2048 + l32 * 64 + ((g ^ s) * 16));
            rd[1] = (uint32_t)(j0 * 2048 + l32 * 64 + (((2 + g) ^ s) * 16));
        } else {
            const int r = (lane & 15) >> 2, t = lane & 3, u = (lane >> 4) & 1, g = lane >> 5;
#pragma unroll
            for (int i = 0; i < W; ++i)
                rd[i] = (uint32_t)((8 * g + r) * ROWS * 2 + 64 * ((j0 + i) ^ r) + (2 * u + (t >> 1)) * 16 + (t & 1) * 8);
        }
    }
    static constexpr int NRD(int W) { return ROW_CONTIG ? W : 2; }

    // operand (tile t of the wave, k-step kk) from the stage at LDS byte offset `base`
    __device__ __forceinline__ static bf16x8 operand(const char* lds, uint32_t base, const uint32_t* rd, int t, int kk) {
        if (!ROW_CONTIG) return *reinterpret_cast<const bf16x8*>(lds + base + rd[kk] + t * 2048);
        const uint16_t* p = reinterpret_cast<const uint16_t*>(lds + base + rd[t] + kk * 16 * ROWS * 2);
        return lds_operand_tr(p, 4 * ROWS);
    }
};

// GM x GN waves, each WM x WN MFMA tiles: work-group tile (32 WM GM) x (32 WN GN).
template <bool A_MCONTIG, bool B_NCONTIG, int GM, int GN, int WM, int WN, int NS, bool F16>
__global__ __launch_bounds__(512, 1) void gemm_kernel(const GemmParams p) {
    using E = Elt<F16>;
    static_assert(GM * GN == 8, "8 waves");
    constexpr int TM = 32 * WM * GM, TN = 32 * WN * GN;
    using RA = Region<A_MCONTIG, TM>;
    using RB = Region<B_NCONTIG, TN>;
    constexpr int STAGE = RA::BYTES + RB::BYTES;
    constexpr int LPG = (RA::CHUNKS + RB::CHUNKS) / 8;     // loads per wave per stage
    constexpr int LPG_A = RA::CHUNKS / 8;
    static_assert(RA::CHUNKS % 8 == 0 && RB::CHUNKS % 8 == 0, "chunks split evenly over 8 waves");
    constexpr int NRA = RA::NRD(WM), NRB = RB::NRD(WN);
    __shared__ __attribute__((aligned(1024))) char lds[NS * STAGE];

    const int wid0 = p.m_order ? (int)blockIdx.x : xcd_remap(blockIdx.x, p.total_wg);
    if (wid0 >= p.total_wg) return;
    const int nks = p.k_splits > 1 ? p.k_splits : 1;
    const int ksp = wid0 % nks;
    const int wid = wid0 / nks;
    const int tn = wid % p.tiles_n;
    const int t1 = wid / p.tiles_n;
    int tm, z, t2 = 0;
    if (p.m_order) {
        // M tiles with their own contraction ranges, ranked by length: the ids walk the ranking
        // (the inner batch index fastest), so the hardware's in-order hand-out of work-groups
        // starts the longest first, on every XCD alike
        const int item = p.m_order[t1 / p.batch_inner];
        tm = item % p.tiles_m;
        z = (item / p.tiles_m) * p.batch_inner + t1 % p.batch_inner;
    } else {
        tm = t1 % p.tiles_m;
        t2 = t1 / p.tiles_m;
        // the outer batch index (the sample, where there is one) varies fastest over the ids, so that
        // every XCD's contiguous id range holds work of all samples (ragged ones differ in length)
        const int zr = t2 % p.nbatch;
        const int n_outer = p.nbatch / p.batch_inner;
        z = (zr % n_outer) * p.batch_inner + zr / n_outer;
    }
    const GemmProblem& pr = p.prob[t2 / p.nbatch];
    const int m0 = tm * TM, n0 = tn * TN;
    const int zo = z / p.batch_inner, zi = z % p.batch_inner;
    const int64_t a_off = (int64_t)z * p.a_batch;
    const int64_t b_off = zo * p.b_outer + (zi / p.b_group) * p.b_inner;
    uint16_t* const Cz = pr.C + zo * p.c_outer + zi * p.c_inner;
    int klen0 = pr.K[0];
    if (p.k_len) klen0 = min(klen0, p.k_len[zo]);
    int k_lo = 0;                                   // start of this work-group's k range
    if (nks > 1) { k_lo = ksp * p.k_split_len; klen0 = min(klen0, k_lo + p.k_split_len); }
    if (p.k_range) {
        const int32_t* kr = p.k_range + ((int64_t)zo * p.tiles_m + tm) * 2;
        k_lo = max(k_lo, kr[0]);
        klen0 = min(klen0, kr[1]);
    }
    klen0 = max(0, klen0 - k_lo);
    const int s_lo = k_lo / BK;                    // first stage of this work-group's k range
    const int klen1 = pr.nseg > 1 ? pr.K[1] : 0;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int set = wave >> 2;
    const int wm = wave % GM, wn = wave / GM;
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds;

    // ---- global -> LDS: this wave's LPG chunks of every stage
    const int64_t lda = pr.lda[0], ldb = pr.ldb[0];
    uint32_t voff[LPG];
    int kpos[LPG];
#pragma unroll
    for (int j = 0; j < LPG; ++j) {
        const int ch = wave + 8 * j;
        if (j < LPG_A) voff[j] = RA::src(ch, lane, m0, p.M_ld, lda, p.a_tiled_m, kpos[j]);
        else voff[j] = RB::src(ch - RA::CHUNKS, lane, n0, p.N, ldb, 0, kpos[j]);
    }
    const char* abase[2];
    const char* bbase[2];
#pragma unroll
    for (int sg = 0; sg < 2; ++sg) {
        const int ss = sg < pr.nseg ? sg : 0;
        abase[sg] = reinterpret_cast<const char*>(pr.A[ss] + a_off);
        if (!p.a_tiled_m) abase[sg] += (A_MCONTIG ? (int64_t)m0 : (int64_t)m0 * lda) * 2;
        bbase[sg] = reinterpret_cast<const char*>(pr.Bm[ss] + b_off) + (B_NCONTIG ? (int64_t)n0 : (int64_t)n0 * ldb) * 2;
    }
    const int64_t a_kstride = A_MCONTIG ? lda * BK * 2 : BK * 2;   // bytes per stage (untiled)
    const int64_t b_kstride = B_NCONTIG ? ldb * BK * 2 : BK * 2;
    const int steps0 = (klen0 + BK - 1) / BK;
    const int steps = steps0 + (klen1 + BK - 1) / BK;

    auto issue = [&](int s) {     // loads of stage s into ring slot s % NS
        const int sg = s >= steps0 ? 1 : 0;
        const int kr = sg ? s - steps0 : s;            // stage inside this work-group's range
        const int krem = (sg ? klen1 : klen0) - kr * BK;
        const int ks = sg ? kr : kr + s_lo;            // stage inside the operand
        const char* ab = abase[sg] + ks * a_kstride;
        if (A_MCONTIG && p.a_tiled_m)   // tiled A: [k / 128][m / 32][128 k][32 m]
            ab = abase[sg] + ((int64_t)(ks >> 2) * p.a_tiled_m * 4096 + (ks & 3) * (BK * 32)) * 2;
        const char* bb = bbase[sg] + ks * b_kstride;
        const uint32_t slot = lds0 + (uint32_t)(s % NS) * STAGE + (uint32_t)wave * 1024u;
        if (krem >= BK) {
#pragma unroll
            for (int j = 0; j < LPG; ++j)
                dma16(j < LPG_A ? ab : bb, voff[j], slot + (j < LPG_A ? j * 8192 : RA::BYTES + (j - LPG_A) * 8192));
        } else {
            const char* zc = reinterpret_cast<const char*>(zero_chunk);
#pragma unroll
            for (int j = 0; j < LPG; ++j) {
                const char* src = (j < LPG_A ? ab : bb) + voff[j];
                dma16_addr(kpos[j] < krem ? src : zc, slot + (j < LPG_A ? j * 8192 : RA::BYTES + (j - LPG_A) * 8192));
            }
        }
    };

    // ---- LDS -> registers
    uint32_t rda[NRA], rdb[NRB];
    RA::template read_offsets<WM>(rda, WM * wm, lane);
    RB::template read_offsets<WN>(rdb, WN * wn, lane);

    f32x16 acc[WN][WM];   // [n tile][m tile]
#pragma unroll
    for (int a = 0; a < WN; ++a)
#pragma unroll
        for (int b = 0; b < WM; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

    // The 256 x 256 bf16 tile with A stored [m][k] and whole stages only (the K/V projection and
    // dX_vis) takes the hand-scheduled loop of gen_gemm_loop.py, one run per contraction segment; every
    // other case takes the ping-pong loop below.
    constexpr bool FAST = !F16 && !A_MCONTIG && GM == 2 && GN == 4 && WM == 4 && WN == 2 && NS == 4;
    if constexpr (FAST) {
        const int st0 = klen0 / BK, st1 = klen1 / BK;
        const bool whole = klen0 % BK == 0 && klen1 % BK == 0 && st0 % 4 == 0 && st1 % 4 == 0 && st0 >= 8 &&
                           (st1 == 0 || st1 >= 8);
        if (whole) {
            uint32_t ra[4], rb[4];
            ra[0] = lds0 + rda[0]; ra[1] = lds0 + rda[1]; ra[2] = ra[0] + 65536u; ra[3] = ra[1] + 65536u;
            rb[0] = lds0 + rdb[0]; rb[1] = lds0 + rdb[1]; rb[2] = rb[0] + 65536u; rb[3] = rb[1] + 65536u;
            const uint32_t lds_w = uniform32(lds0 + (uint32_t)wave * 1024u);
            for (int sg = 0; sg < (st1 ? 2 : 1); ++sg) {
                const int nst = sg ? st1 : st0;
                const char* ap = uniform_ptr(abase[sg] + (int64_t)(sg ? 0 : s_lo) * a_kstride);
                const char* bp = uniform_ptr(bbase[sg] + (int64_t)(sg ? 0 : s_lo) * b_kstride);
                int trips = uniform32(nst / 4), todo = uniform32(nst);
                __syncthreads();     // the stage buffers are free
                if (B_NCONTIG) {
                    asm volatile(
#include "lvx_gemm_loop_bt.inc"
                        : "+{v[0:15]}"(acc[0][0]), "+{v[16:31]}"(acc[0][1]), "+{v[32:47]}"(acc[0][2]), "+{v[48:63]}"(acc[0][3]),
                          "+{v[64:79]}"(acc[1][0]), "+{v[80:95]}"(acc[1][1]), "+{v[96:111]}"(acc[1][2]), "+{v[112:127]}"(acc[1][3]),
                          "+{s[44:45]}"(ap), "+{s[46:47]}"(bp), "+{s51}"(trips), "+{s52}"(todo)
                        : "{v224}"(ra[0]), "{v225}"(ra[1]), "{v226}"(ra[2]), "{v227}"(ra[3]),
                          "{v228}"(rb[0]), "{v229}"(rb[1]), "{v230}"(rb[2]), "{v231}"(rb[3]),
                          "{v232}"(voff[0]), "{v233}"(voff[1]), "{v234}"(voff[2]), "{v235}"(voff[3]),
                          "{s48}"(uniform32((uint32_t)a_kstride)), "{s49}"(uniform32((uint32_t)b_kstride)), "{s50}"(lds_w)
                        : "memory", "vcc", "scc", "m0", "s53", "s54", "s55", LVX_GEMM_LOOP_CLOBBERS);
                } else {
                    asm volatile(
#include "lvx_gemm_loop_bp.inc"
                        : "+{v[0:15]}"(acc[0][0]), "+{v[16:31]}"(acc[0][1]), "+{v[32:47]}"(acc[0][2]), "+{v[48:63]}"(acc[0][3]),
                          "+{v[64:79]}"(acc[1][0]), "+{v[80:95]}"(acc[1][1]), "+{v[96:111]}"(acc[1][2]), "+{v[112:127]}"(acc[1][3]),
                          "+{s[44:45]}"(ap), "+{s[46:47]}"(bp), "+{s51}"(trips), "+{s52}"(todo)
                        : "{v224}"(ra[0]), "{v225}"(ra[1]), "{v226}"(ra[2]), "{v227}"(ra[3]),
                          "{v228}"(rb[0]), "{v229}"(rb[1]), "{v230}"(rb[2]), "{v231}"(rb[3]),
                          "{v232}"(voff[0]), "{v233}"(voff[1]), "{v234}"(voff[2]), "{v235}"(voff[3]),
                          "{s48}"(uniform32((uint32_t)a_kstride)), "{s49}"(uniform32((uint32_t)b_kstride)), "{s50}"(lds_w)
                        : "memory", "vcc", "scc", "m0", "s53", "s54", "s55", LVX_GEMM_LOOP_CLOBBERS);
                }
            }
            goto epilogue;
        }
    }

    // prologue: stages 0 .. NS-2 in flight, stage 0 landed
#pragma unroll
    for (int s = 0; s < NS - 1; ++s)
        if (s < steps) issue(s);
    if (steps > NS - 2) wait_vmcnt<(NS - 2) * LPG>();
    else wait_vmcnt<0>();
    phase_barrier();
    if (set == 1) phase_barrier();        // waves 4-7 run half a stage behind waves 0-3

    for (int s = 0; s < steps; ++s) {
        // memory phase: request stage s+NS-1, fetch this wave's operands of stage s
        if (s + NS - 1 < steps) issue(s + NS - 1);
        const uint32_t base = (uint32_t)(s % NS) * STAGE;
        bf16x8 am[2][WM], bn[2][WN];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
            for (int t = 0; t < WM; ++t) am[kk][t] = RA::operand(lds, base, rda, t, kk);
#pragma unroll
            for (int t = 0; t < WN; ++t) bn[kk][t] = RB::operand(lds, base + RA::BYTES, rdb, t, kk);
        }
        wait_lds();     // the slot may be overwritten once the next barrier is passed
        if (set == 1) {                     // stage s+1 must have landed before waves 0-3 read it
            if (s + NS - 1 < steps) wait_vmcnt<(NS - 2) * LPG>();
            else wait_vmcnt<0>();
        }
        phase_barrier();
        // compute phase
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int nt = 0; nt < WN; ++nt)
#pragma unroll
                for (int mt = 0; mt < WM; ++mt) acc[nt][mt] = E::mfma(bn[kk][nt], am[kk][mt], acc[nt][mt]);
        __builtin_amdgcn_s_setprio(0);
        if (set == 0) {
            if (s + NS - 1 < steps) wait_vmcnt<(NS - 2) * LPG>();
            else wait_vmcnt<0>();
        }
        phase_barrier();
    }
    if (set == 0) phase_barrier();

epilogue:
    // C^T tile: accumulator rows = n, cols = m
    if (nks > 1) {   // partial tile of a split contraction: fp32, into this split's slice
        float* const C32 = p.c32 + ksp * p.c32_split + (int64_t)z * p.c32_batch;
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
#pragma unroll
                        for (int r = 0; r < 4; ++r) C32[(int64_t)(n + r) * p.c32_ld + m] = acc[nt][mt][4 * vg + r];
                    }
                }
        }
        return;
    }
    // A lane holds 4 consecutive columns of one C row, so storing from the registers writes 8
    // bytes per lane into 32 different rows per instruction.  Where 256 rows of the tile fit the
    // stage buffers (free by now) they go through LDS instead, 256 rows at a time, and leave as
    // whole row segments (TN * 2 bytes), 16 bytes per lane.  16-byte chunk c of row r sits at
    // position c ^ (r mod chunks per row), with its two 8-byte halves exchanged in rows where
    // bits 3 and 4 differ: the 32 rows a half-wave's 8-byte writes touch then land in different
    // chunks or, where they share a chunk position or banks (positions 8 or 16 apart), in
    // different halves; a read instruction takes whole rows.  Both are conflict-free.
    // `pair(mt, nt, vg)`: the 4 values of accumulator tile (nt, mt), register group vg, as two
    // packed words.
    constexpr int CPR = TN / 8;                 // 16-byte chunks per row
    constexpr bool VIA_LDS = (TN == 256 || TN == 128) && TM % 256 == 0 && 256 * TN * 2 <= NS * STAGE;
    auto store_via_lds = [&](auto pair, uint16_t* dst) __attribute__((always_inline)) {
#pragma unroll
        for (int pass = 0; pass < TM / 256; ++pass) {
            __syncthreads();                    // every wave is done with what the buffers held
#pragma unroll
            for (int mt = 0; mt < WM; ++mt) {
                if (((WM * wm + mt) >> 3) != pass) continue;
#pragma unroll
                for (int nt = 0; nt < WN; ++nt)
#pragma unroll
                    for (int vg = 0; vg < 4; ++vg) {
                        const int ml = 32 * ((WM * wm + mt) & 7) + l32;
                        const int c = 4 * (WN * wn + nt) + vg;
                        *reinterpret_cast<u32x2*>(lds + ml * (TN * 2) + ((c ^ (l32 & (CPR - 1))) << 4) +
                                                  ((g ^ ((l32 >> 3) & 1) ^ (l32 >> 4)) << 3)) = pair(mt, nt, vg);
                    }
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < CPR / 2; ++i) {
                const int row = i * (512 / CPR) + tid / CPR, cc = tid % CPR;
                u32x4 val = *reinterpret_cast<const u32x4*>(lds + row * (TN * 2) + ((cc ^ (row & (CPR - 1))) << 4));
                if (((row >> 3) ^ (row >> 4)) & 1) val = u32x4{val[2], val[3], val[0], val[1]};
                const int m = m0 + 256 * pass + row, n = n0 + cc * 8;
                // (a streaming store: nobody on this CU reads the tile again)
                if (m < p.M && n < p.N) __builtin_nontemporal_store(val, reinterpret_cast<u32x4*>(dst + (int64_t)m * pr.ldc + n));
            }
        }
    };
    if (p.norm_w && t2 / p.nbatch == 0) {
        // RMS norm over each 128-column group (N and the tile are multiples of 128): the
        // group's columns sit in HW = 4 / WN waves with consecutive wn; row sums of squares
        // are exchanged through LDS, which no wave reads any more.
        constexpr int HW = 4 / WN;
        static_assert(WN == 2 || WN == 4, "a 128-column group spans 1 or 2 waves");
        float* const red = reinterpret_cast<float*>(lds);
        float rs[WM];
#pragma unroll
        for (int mt = 0; mt < WM; ++mt) {
            float ss = 0.f;
#pragma unroll
            for (int nt = 0; nt < WN; ++nt)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float x = E::hi(E::pack(0.f, acc[nt][mt][i]));   // the product as bf16
                    acc[nt][mt][i] = x;
                    ss = fmaf(x, x, ss);
                }
            ss += __shfl_xor(ss, 32);
            rs[mt] = ss;
            if (HW > 1 && g == 0) red[(wave * WM + mt) * 32 + l32] = ss;
        }
        if (HW > 1) {
            __syncthreads();
            const int pw = wm + GM * (wn ^ 1);
#pragma unroll
            for (int mt = 0; mt < WM; ++mt) rs[mt] += red[(pw * WM + mt) * 32 + l32];
        }
        const int groups = p.N >> 7;
        if (VIA_LDS) {       // (N is a multiple of 128 here)
            float rr[WM];
#pragma unroll
            for (int mt = 0; mt < WM; ++mt) {
                const int m = m0 + 32 * (WM * wm + mt) + l32;
                rr[mt] = rsqrtf(rs[mt] * (1.f / 128.f) + p.norm_eps);
                const int ncol = n0 + 32 * WN * wn;
                if (m < p.M && p.rstd && g == 0 && (wn & (HW - 1)) == 0 && ncol < p.N) p.rstd[(int64_t)m * groups + (ncol >> 7)] = rr[mt];
            }
            if (p.c_raw)
                store_via_lds([&](int mt, int nt, int vg) {
                    u32x2 w;
                    w[0] = E::pack(acc[nt][mt][4 * vg], acc[nt][mt][4 * vg + 1]);
                    w[1] = E::pack(acc[nt][mt][4 * vg + 2], acc[nt][mt][4 * vg + 3]);
                    return w;
                }, p.c_raw + (Cz - pr.C));
            store_via_lds([&](int mt, int nt, int vg) {
                const int n = 32 * (WN * wn + nt) + 8 * vg + 4 * g;       // n0 is a multiple of 128
                const u32x2 wt = *reinterpret_cast<const u32x2*>(p.norm_w + (n & 127));
                const float r = rr[mt];
                const u32x2 h = {E::pack(acc[nt][mt][4 * vg] * r, acc[nt][mt][4 * vg + 1] * r),
                                 E::pack(acc[nt][mt][4 * vg + 2] * r, acc[nt][mt][4 * vg + 3] * r)};
                u32x2 y;
                y[0] = E::pack(E::lo(wt[0]) * E::lo(h[0]), E::hi(wt[0]) * E::hi(h[0]));
                y[1] = E::pack(E::lo(wt[1]) * E::lo(h[1]), E::hi(wt[1]) * E::hi(h[1]));
                return y;
            }, Cz);
            return;
        }
#pragma unroll
        for (int mt = 0; mt < WM; ++mt) {
            const int m = m0 + 32 * (WM * wm + mt) + l32;
            if (m >= p.M) continue;
            const float r = rsqrtf(rs[mt] * (1.f / 128.f) + p.norm_eps);
            const int ncol = n0 + 32 * WN * wn;
            if (p.rstd && g == 0 && (wn & (HW - 1)) == 0 && ncol < p.N) p.rstd[(int64_t)m * groups + (ncol >> 7)] = r;
#pragma unroll
            for (int nt = 0; nt < WN; ++nt)
#pragma unroll
                for (int vg = 0; vg < 4; ++vg) {
                    const int n = n0 + 32 * (WN * wn + nt) + 8 * vg + 4 * g;
                    if (n < p.N) {
                        const float a[4] = {acc[nt][mt][4 * vg], acc[nt][mt][4 * vg + 1], acc[nt][mt][4 * vg + 2], acc[nt][mt][4 * vg + 3]};
                        if (p.c_raw) {
                            u32x2 w;
                            w[0] = E::pack(a[0], a[1]);
                            w[1] = E::pack(a[2], a[3]);
                            *reinterpret_cast<u32x2*>(p.c_raw + (Cz - pr.C) + (int64_t)m * pr.ldc + n) = w;
                        }
                        const u32x2 wt = *reinterpret_cast<const u32x2*>(p.norm_w + (n & 127));
                        const u32x2 h = {E::pack(a[0] * r, a[1] * r), E::pack(a[2] * r, a[3] * r)};
                        u32x2 y;
                        y[0] = E::pack(E::lo(wt[0]) * E::lo(h[0]), E::hi(wt[0]) * E::hi(h[0]));
                        y[1] = E::pack(E::lo(wt[1]) * E::lo(h[1]), E::hi(wt[1]) * E::hi(h[1]));
                        *reinterpret_cast<u32x2*>(Cz + (int64_t)m * pr.ldc + n) = y;
                    }
                }
        }
        return;
    }
    if (VIA_LDS && (p.N & 7) == 0) {
        store_via_lds([&](int mt, int nt, int vg) {
            u32x2 w;
            w[0] = E::pack(acc[nt][mt][4 * vg], acc[nt][mt][4 * vg + 1]);
            w[1] = E::pack(acc[nt][mt][4 * vg + 2], acc[nt][mt][4 * vg + 3]);
            return w;
        }, Cz);
        return;
    }
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
                    w[0] = E::pack(acc[nt][mt][4 * vg], acc[nt][mt][4 * vg + 1]);
                    w[1] = E::pack(acc[nt][mt][4 * vg + 2], acc[nt][mt][4 * vg + 3]);
                    *reinterpret_cast<u32x2*>(Cz + (int64_t)m * pr.ldc + n) = w;
                }
            }
    }
}

template <int GM, int GN, int WM, int WN, int NS, bool F16>
hipError_t launch_cfg_t(const GemmParams& p, int grid, bool a_mcontig, bool b_ncontig, hipStream_t st) {
    if (!a_mcontig && !b_ncontig)
        return launch1((gemm_kernel<false, false, GM, GN, WM, WN, NS, F16>), dim3(grid), dim3(512), st, p);
    else if (!a_mcontig && b_ncontig)
        return launch1((gemm_kernel<false, true, GM, GN, WM, WN, NS, F16>), dim3(grid), dim3(512), st, p);
    else if (a_mcontig && !b_ncontig)
        return launch1((gemm_kernel<true, false, GM, GN, WM, WN, NS, F16>), dim3(grid), dim3(512), st, p);
    else
        return launch1((gemm_kernel<true, true, GM, GN, WM, WN, NS, F16>), dim3(grid), dim3(512), st, p);
}

template <int GM, int GN, int WM, int WN, int NS>
hipError_t launch_cfg(GemmParams p, bool a_mcontig, bool b_ncontig, hipStream_t st) {
    constexpr int TM = 32 * WM * GM, TN = 32 * WN * GN;
    p.tiles_m = (p.M + TM - 1) / TM;
    p.tiles_n = (p.N + TN - 1) / TN;
    p.total_wg = p.nprob * p.nbatch * p.tiles_m * p.tiles_n * (p.k_splits > 1 ? p.k_splits : 1);
    const int grid = ((p.total_wg + 7) / 8) * 8;
    if (p.f16) return launch_cfg_t<GM, GN, WM, WN, NS, true>(p, grid, a_mcontig, b_ncontig, st);
    return launch_cfg_t<GM, GN, WM, WN, NS, false>(p, grid, a_mcontig, b_ncontig, st);
}

}  // namespace

// Work-group tile by shape: 256 x 256 in general; for a narrow C (N <= 128, the
// dQ GEMM) 512 x 128, or 256 x 128 when there are not 512 rows or when M tiles have
// their own contraction ranges (k_range is kept per 256 rows: finer ranges skip more).
hipError_t launch_gemm(const GemmParams& p, bool a_mcontig, bool b_ncontig, hipStream_t st) {
    for (int i = 0; i < p.nprob; ++i) {
        const GemmProblem& pr = p.prob[i];
        // all problems and both contraction segments share the per-thread load offsets
        if (pr.lda[0] != p.prob[0].lda[0] || pr.ldb[0] != p.prob[0].ldb[0]) return hipErrorInvalidValue;
        if (pr.nseg > 1 && (pr.lda[1] != pr.lda[0] || pr.ldb[1] != pr.ldb[0])) return hipErrorInvalidValue;
    }
    if (p.N > 128) return launch_cfg<2, 4, 4, 2, 4>(p, a_mcontig, b_ncontig, st);
    if (p.m_order && (!p.k_range || p.nprob != 1 || p.k_splits > 1 || p.N > 128)) return hipErrorInvalidValue;
    if (p.M > 256 && !p.k_range) return launch_cfg<8, 1, 2, 4, 3>(p, a_mcontig, b_ncontig, st);
    return launch_cfg<4, 2, 2, 2, 4>(p, a_mcontig, b_ncontig, st);
}

}  // namespace lvx
