// Flash cross-attention forward for gfx950: one launch computes, for a window
// of text rows, O = softmax(scale * Q K^T) V (bf16) and the per-row natural-log
// LSE against the local K/V shard (or one key split of it).
//
// Mapping.  A work-group is 4 wavefronts.  Each wavefront owns 32 text rows of
// ONE q head; the 4 waves of a group cover the q heads that share a kv head
// (G = 4: four heads x 32 rows; G = 1: one head x 128 rows), so the K/V tile
// staged in LDS is read by the whole GQA group and nothing is expanded in HBM.
// (The bf16 kernel without a dense bias or an interval mask, fwd_kernel_pipe, also has a wide form in which
// a wavefront owns 64 rows; see there.)
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
// K and V tiles ([64 keys][128] bf16, 16 KiB each) go from global memory
// straight into LDS with global_load_lds_dwordx4, double-buffered: tile t+1 is
// in flight while tile t is consumed, one barrier per tile, no staging
// registers and no LDS stores.  That load writes 64 lanes x 16 bytes
// contiguously, so rows cannot be padded; instead the 16-byte chunk c of row r
// is kept at position c ^ f(r), f(r) = ((r & 3) << 2) | ((r >> 2) & 3): the 16
// rows a 16-byte operand read of K touches land in 16 different positions, and
// the 4 rows a transposing read of V touches land in 4 different 64-byte
// groups - both conflict-free.  Loads past the end of the key range are
// clamped to its last row (those keys are masked out of S).
#include "lvx_common.hpp"
#include "lvx_kernels.hpp"

namespace lvx {

namespace {

constexpr int D = 128;
constexpr int BN = 64;        // keys per tile
constexpr int TILE_BYTES = BN * D * 2;
constexpr int BIG = 0x3fffffff;
constexpr float RESCALE_LOG2 = 8.f;
constexpr float LOG2E_F = 1.4426950408889634f, LN2_F = 0.6931471805599453f;

// BIAS: a dense fp32 bias is added to scale * S before the softmax; the scores are
// then carried in log2 units (S*c + bias*log2e) instead of raw.
// DH: head dimension, 16, 32, 64 or 128.  The LDS tiles keep their 256-byte rows and chunk
// permutation whatever DH is: below 128 only the first DH / 8 chunks of a row hold data (the
// lanes that would load the others repeat a chunk of the same row), and the k-steps of S^T and
// the 32-wide blocks of O^T past DH do not exist.  With 16 the one block of O^T is half real:
// its upper 16 rows are products with those repeated chunks and are never stored.
template <int DH, bool MASKED, bool BIAS, bool F16>
__global__ __launch_bounds__(256, 2) void fwd_kernel(const FwdParams p) {
    using E = Elt<F16>;
    static_assert(DH == 16 || DH == 32 || DH == 64 || DH == 128, "head dimension");
    constexpr int NKK = DH / 16, NDT = DH >= 32 ? DH / 32 : 1;
    __shared__ __attribute__((aligned(1024))) char kv_lds[2][2][TILE_BYTES];   // [buffer][K, V]
    __shared__ int red[4][4];

    const int wid = xcd_remap(blockIdx.x, p.total_wg);
    if (wid >= p.total_wg) return;
    const int tile = wid % p.n_row_tiles;
    const int t1 = wid / p.n_row_tiles;
    const int split = t1 % p.nsplit;
    const int t2 = t1 / p.nsplit;
    // samples vary faster than head groups: every XCD (a contiguous range of ids) then gets
    // work-groups of all samples, and ragged samples do not leave some XCDs idle early
    const int b = t2 % p.B;
    const int hg = t2 / p.B;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l32 = lane & 31, g = lane >> 5;
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
    // the same in every lane of the work-group: keep them in scalar registers
    lo = __builtin_amdgcn_readfirstlane(lo);
    hi = __builtin_amdgcn_readfirstlane(hi);
    in_lo = __builtin_amdgcn_readfirstlane(in_lo);
    in_hi = __builtin_amdgcn_readfirstlane(in_hi);

    // Q^T as B operand, resident for the whole kernel
    bf16x8 qreg[NKK];
    {
        const uint16_t* qp = p.q + b * p.qs.b + h * p.qs.h + (int64_t)row * p.qs.s + g * 8;
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk) qreg[kk] = as_bf16x8(ldg16(qp + kk * 16, row_ok));
    }

    const char* kbase = reinterpret_cast<const char*>(p.k + b * p.ks.b + hk * p.ks.h);
    const char* vbase = reinterpret_cast<const char*>(p.v + b * p.vs.b + hk * p.vs.h);
    const uint32_t krow_b = (uint32_t)p.ks.s * 2u, vrow_b = (uint32_t)p.vs.s * 2u;   // bytes per key row

    // global -> LDS: wave w moves the 1 KiB chunks w, w+4, w+8, w+12 (4 rows each)
    // of the K tile and of the V tile; lane i fills position i & 15 of row i >> 4.
    const int wave_u = wave;
    const int ld_r = lane >> 4;
    const uint32_t ld_c = (uint32_t)(((lane & 15) ^ ((ld_r << 2) | wave_u)) & (DH / 8 - 1)) * 16u;   // chunk this lane fetches
    const uint32_t lds0 = (uint32_t)(uintptr_t)&kv_lds[0][0][0];
    auto issue = [&](int kv0, int buf) {
        const char* kb = kbase + (int64_t)kv0 * krow_b;
        const char* vb = vbase + (int64_t)kv0 * vrow_b;
        const uint32_t slot = lds0 + (uint32_t)buf * (2 * TILE_BYTES) + (uint32_t)wave_u * 1024u;
        const int last = kv_hi - 1 - kv0;          // rows past `last` repeat it
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t r = (uint32_t)min(4 * (wave_u + 4 * j) + ld_r, last);
            dma16(kb, r * krow_b + ld_c, slot + j * 4096);
            dma16(vb, r * vrow_b + ld_c, slot + TILE_BYTES + j * 4096);
        }
    };

    // LDS -> operands.  K rows (A of S^T): 16 bytes at row * 256 + ((2 kk + g) ^ f(row)) * 16.
    const int f_row = ((l32 & 3) << 2) | ((l32 >> 2) & 3);
    const uint32_t k_rd = (uint32_t)(l32 * 256), k_h = (uint32_t)((g ^ f_row) << 4);
    // V^T (A of O^T += V^T P^T), keys in accumulator order: first half rows 16 j + 4 g + r,
    // second half 8 rows further down, whose f differs in bit 1.
    uint32_t v_rd[4][2];
    {
        const int r = (lane & 15) >> 2, t = lane & 3, u = (lane >> 4) & 1;
        const int low = (2 * u + (t >> 1)) ^ g;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
            v_rd[dt][0] = (uint32_t)((4 * g + r) * 256 + (4 * (dt ^ r) + low) * 16 + (t & 1) * 8);
            v_rd[dt][1] = (uint32_t)((4 * g + r + 8) * 256 + (4 * (dt ^ r) + (low ^ 2)) * 16 + (t & 1) * 8);
        }
    }

    f32x16 acc[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[dt][v] = 0.f;
    float m_i = -INFINITY, l_i = 0.f;
    const float c = p.scale_log2e;
    const float cc = BIAS ? 1.f : c;              // factor from the carried scores to log2 units
    const float* brow = nullptr;                  // this lane's row of the bias
    if (BIAS) brow = p.bias + b * p.bias_b + h * p.bias_h + (int64_t)min(row, p.row_end - 1) * p.bias_r;

    const int t_begin = (hi > lo) ? lo / BN : 0;
    const int t_end = (hi > lo) ? (hi + BN - 1) / BN : 0;
    if (t_end > t_begin) issue(t_begin * BN, 0);

    for (int t = t_begin; t < t_end; ++t) {
        const int kv0 = t * BN;
        const int buf = (t - t_begin) & 1;
        const char* Ks = kv_lds[buf][0];
        const char* Vs = kv_lds[buf][1];

        // tile t has landed (this wave's part: vmcnt; everyone's: barrier); the
        // barrier also says every wave is done reading tile t-1, whose buffer
        // the loads of tile t+1 may now overwrite
        wait_vmcnt<0>();
        __syncthreads();
        if (t + 1 < t_end) issue(kv0 + BN, buf ^ 1);

        // S^T = K Q^T : rows = keys (two 32-key sub-tiles), cols = text rows.
        // All 16 K operands are requested before the first MFMA, so the LDS
        // latency is paid once per tile and not once per k-step.
        bf16x8 ka[NKK][2];
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk) {
            const char* kp = Ks + k_rd + ((uint32_t)(kk * 32) ^ k_h);
            ka[kk][0] = *reinterpret_cast<const bf16x8*>(kp);
            ka[kk][1] = *reinterpret_cast<const bf16x8*>(kp + 32 * 256);
        }
        __builtin_amdgcn_sched_barrier(0);
        f32x16 s0, s1;
#pragma unroll
        for (int v = 0; v < 16; ++v) { s0[v] = 0.f; s1[v] = 0.f; }
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk) {
            s0 = E::mfma(ka[kk][0], qreg[kk], s0);
            s1 = E::mfma(ka[kk][1], qreg[kk], s1);
        }
        __builtin_amdgcn_sched_barrier(0);
        // V^T operands of this tile: requested now, they land during the softmax
        u32x2 va[NDT][4][2];
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                va[dt][j][0] = lds_read_tr16(reinterpret_cast<const uint16_t*>(Vs + v_rd[dt][0] + j * 4096));
                va[dt][j][1] = lds_read_tr16(reinterpret_cast<const uint16_t*>(Vs + v_rd[dt][1] + j * 4096));
            }
        __builtin_amdgcn_sched_barrier(0);

        if (BIAS) {
            // register group vg of lane-half g holds keys kv0 + 8 vg + 4 g + 0..3 (+32 for s1);
            // groups past the end re-read the last one (those keys are masked below)
#pragma unroll
            for (int vg = 0; vg < 4; ++vg) {
                const int k0 = kv0 + 8 * vg + 4 * g;
                const f32x4 ba = *reinterpret_cast<const f32x4*>(brow + min(k0, (p.Lkv - 1) & ~3));
                const f32x4 bb = *reinterpret_cast<const f32x4*>(brow + min(k0 + 32, (p.Lkv - 1) & ~3));
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    s0[4 * vg + r] = fmaf(s0[4 * vg + r], c, ba[r] * LOG2E_F);
                    s1[4 * vg + r] = fmaf(s1[4 * vg + r], c, bb[r] * LOG2E_F);
                }
            }
        }

        if (kv0 < in_lo || kv0 + BN > in_hi) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int kv = kv0 + acc_row(v, g);
                if (kv < my_s || kv >= my_e) s0[v] = -INFINITY;
                if (kv + 32 < my_s || kv + 32 >= my_e) s1[v] = -INFINITY;
            }
        }

        float mx = max3(s0[0], s1[0], s0[1]);
        mx = max3(mx, s1[1], s0[2]);
#pragma unroll
        for (int v = 3; v < 16; v += 1) mx = max3(mx, s1[v - 1], s0[v]);
        mx = fmaxf(mx, s1[15]);
        {   // other half of the wave holds the other 32 keys of the same text row
            const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
            mx = max3(__uint_as_float(sw[0]), __uint_as_float(sw[1]), m_i);
        }
        // Lazy rescale: the reference point m_i of a row only moves when the row
        // maximum has grown by more than 2^RESCALE_LOG2 since it was set, so P may
        // reach 2^RESCALE_LOG2 instead of 1 (harmless in fp32 / bf16) and the
        // rescale of O happens a few times per row instead of almost every tile.
        const float mcand = mx * cc;                      // mx >= m_i
        const float m_ic = m_i * cc;
        const bool move = (mx != -INFINITY) && !(mcand - m_ic <= RESCALE_LOG2);
        const float alpha = move ? __builtin_amdgcn_exp2f(m_ic - mcand) : 1.f;
        if (move) m_i = mx;
        const float mc = (m_i == -INFINITY) ? 0.f : m_i * cc;

        // P^T as B operand: k-step j covers keys 16j..16j+15 of the tile.  The row
        // sum is taken in fp32 before the rounding to bf16 (summing the rounded
        // values would put the LSE off by up to a bf16 ulp of the largest term).
        bf16x8 pb[4];
        float rs0 = 0.f, rs1 = 0.f;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            u32x4 u0, u1;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int v = 8 * j + 2 * e;
                const float a0 = __builtin_amdgcn_exp2f(fmaf(s0[v], cc, -mc)), a1 = __builtin_amdgcn_exp2f(fmaf(s0[v + 1], cc, -mc));
                const float b0 = __builtin_amdgcn_exp2f(fmaf(s1[v], cc, -mc)), b1 = __builtin_amdgcn_exp2f(fmaf(s1[v + 1], cc, -mc));
                rs0 += a0 + a1;
                rs1 += b0 + b1;
                u0[e] = E::pack(a0, a1);
                u1[e] = E::pack(b0, b1);
            }
            pb[j] = as_bf16x8(u0);
            pb[2 + j] = as_bf16x8(u1);
        }
        l_i = l_i * alpha + (rs0 + rs1);

        if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {   // the running max moved for some row
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[dt][v] *= alpha;
        }

        // O^T += V^T P^T
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const u32x4 a = {va[dt][j][0][0], va[dt][j][0][1], va[dt][j][1][0], va[dt][j][1][1]};
                acc[dt] = E::mfma(as_bf16x8(a), pb[j], acc[dt]);
            }
    }

    // epilogue: the two lane halves hold partial row sums of the same row
    const float l_tot = l_i + __shfl_xor(l_i, 32);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (row_ok) {
        uint16_t* op = p.o + split * p.o_split_stride + b * p.os.b + h * p.os.h + (int64_t)row * p.os.s;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int vg = 0; vg < 4; ++vg) {
                if (dt * 32 + 8 * vg + 4 * g >= DH) continue;      // only with DH = 16
                u32x2 w;
                w[0] = E::pack(acc[dt][4 * vg] * inv, acc[dt][4 * vg + 1] * inv);
                w[1] = E::pack(acc[dt][4 * vg + 2] * inv, acc[dt][4 * vg + 3] * inv);
                *reinterpret_cast<u32x2*>(op + dt * 32 + 8 * vg + 4 * g) = w;
            }
        if (g == 0) {
            const float lse = l_tot > 0.f ? m_i * (BIAS ? LN2_F : p.scale) + __logf(l_tot) : -INFINITY;
            p.lse[split * p.lse_split_stride + ((int64_t)b * p.Hq + h) * p.lse_bh_stride + row] = lse;
        }
    }
}

// registers the hand-scheduled loop uses besides its operands (see gen_fwd_loop.py)
#define LVX_FWD_LOOP_CLOBBERS "v96", "v97", "v98", "v99", "v100", "v101", "v102", "v103", "v104", "v105", "v106", "v107", "v108", "v109", "v110", "v111", "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120", "v121", "v122", "v123", "v124", "v125", "v126", "v127", "v128", "v129", "v130", "v131", "v132", "v133", "v134", "v135", "v136", "v137", "v138", "v139", "v140", "v141", "v142", "v143", "v144", "v145", "v146", "v147", "v148", "v149", "v150", "v151", "v152", "v153", "v154", "v155", "v156", "v157", "v158", "v159", "v160", "v161", "v162", "v163", "v164", "v165", "v166", "v167", "v168", "v169", "v170", "v171", "v172", "v173", "v174", "v175", "v176", "v177", "v178", "v179", "v180", "v181", "v182", "v183", "v184", "v185", "v186", "v187", "v188", "v189", "v190", "v191", "v192", "v193", "v194", "v195", "v196", "v197", "v198", "v199", "v200", "v201", "v202", "v203", "v204", "v205", "v206", "v207", "v208", "v209", "v210", "v211", "v212", "v213", "v214", "v215", "v246", "v247", "v248", "v249", "v250", "v251", "v252", "v253"

// the same for the wide loop (gen_fwd_loop_wide.py): its working VGPRs and the accumulation registers
#define LVX_FWD_WIDE_CLOBBERS "v192", "v193", "v194", "v195", "v196", "v197", "v198", "v199", "v224", "v225", "v226", "v227", "v228", "v229", "v230", "v231", "v232", "v233", "v234", "v235", "v236", "v237", "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", "a10", "a11", "a12", "a13", "a14", "a15", "a16", "a17", "a18", "a19", "a20", "a21", "a22", "a23", "a24", "a25", "a26", "a27", "a28", "a29", "a30", "a31", "a32", "a33", "a34", "a35", "a36", "a37", "a38", "a39", "a40", "a41", "a42", "a43", "a44", "a45", "a46", "a47", "a48", "a49", "a50", "a51", "a52", "a53", "a54", "a55", "a56", "a57", "a58", "a59", "a60", "a61", "a62", "a63", "a64", "a65", "a66", "a67", "a68", "a69", "a70", "a71", "a72", "a73", "a74", "a75", "a76", "a77", "a78", "a79", "a80", "a81", "a82", "a83", "a84", "a85", "a86", "a87", "a88", "a89", "a90", "a91", "a92", "a93", "a94", "a95", "a96", "a97", "a98", "a99", "a100", "a101", "a102", "a103", "a104", "a105", "a106", "a107", "a108", "a109", "a110", "a111", "a112", "a113", "a114", "a115", "a116", "a117", "a118", "a119", "a120", "a121", "a122", "a123", "a124", "a125", "a126", "a127", "a128", "a129", "a130", "a131", "a132", "a133", "a134", "a135", "a136", "a137", "a138", "a139", "a140", "a141", "a142", "a143", "a144", "a145", "a146", "a147", "a148", "a149", "a150", "a151", "a152", "a153", "a154", "a155", "a156", "a157", "a158", "a159", "a160", "a161", "a162", "a163", "a164", "a165", "a166", "a167", "a168", "a169", "a170", "a171", "a172", "a173", "a174", "a175", "a176", "a177", "a178", "a179", "a180", "a181", "a182", "a183", "a184", "a185", "a186", "a187", "a188", "a189", "a190", "a191"

// The bf16 kernel without a dense bias or an interval mask (the one the benchmarks run): fwd_kernel's mapping, LDS
// layout and tile code, but the run of key tiles that every row of the work-group sees in full
// goes through a hand-scheduled loop (gen_fwd_loop.py) in which every wave interleaves the
// MFMAs of a tile with the exponentials of that tile and the scores of the next one.  The
// tiles before and after that run (the partial last tile, rows past the window) take the plain tile code.
//
// NBLK = 2 is the wide form: a wave owns two blocks of 32 rows of its head (64 rows), has its
// SIMD to itself (one work-group per CU, 512 registers per lane) and feeds every K / V operand it
// reads from LDS to two MFMAs, one per block (gen_fwd_loop_wide.py): half the LDS reads and half
// the global -> LDS bytes per MFMA.
template <int NBLK>
__global__ __launch_bounds__(256, 3 - NBLK) void fwd_kernel_pipe(const FwdParams p) {
    constexpr bool MASKED = false, BIAS = false, F16 = false;
    using E = Elt<F16>;
    __shared__ __attribute__((aligned(1024))) char kv_lds[2][2][TILE_BYTES];   // [buffer][K, V]
    __shared__ int red[4][4];

    const int wid = xcd_remap(blockIdx.x, p.total_wg);
    if (wid >= p.total_wg) return;
    const int tile = wid % p.n_row_tiles;
    const int t1 = wid / p.n_row_tiles;
    const int split = t1 % p.nsplit;
    const int t2 = t1 / p.nsplit;
    // samples vary faster than head groups: every XCD (a contiguous range of ids) then gets
    // work-groups of all samples, and ragged samples do not leave some XCDs idle early
    const int b = t2 % p.B;
    const int hg = t2 / p.B;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int h = hg * p.HG + (wave % p.HG);
    const int hk = h / p.G;
    int row[NBLK];
    bool row_ok[NBLK];
#pragma unroll
    for (int blk = 0; blk < NBLK; ++blk) {
        row[blk] = p.row_begin + ((tile * p.RS + wave / p.HG) * NBLK + blk) * 32 + l32;
        row_ok[blk] = row[blk] < p.row_end;
    }

    int kv_len = p.Lkv;
    if (p.kv_len) kv_len = min(p.kv_len[b], p.Lkv);
    const int kv_lo = split * p.split_len;
    const int kv_hi = min(kv_len, kv_lo + p.split_len);

    // this lane's visible key interval, per row block
    int my_s[NBLK], my_e[NBLK];
    int lo = BIG, hi = 0, in_lo = 0, in_hi = BIG;
#pragma unroll
    for (int blk = 0; blk < NBLK; ++blk) {
        my_s[blk] = kv_lo;
        my_e[blk] = kv_hi;
        if (MASKED) {
            if (row_ok[blk]) {
                my_s[blk] = max(kv_lo, p.kv_start[(int64_t)b * p.Lq + row[blk]]);
                my_e[blk] = min(kv_hi, p.kv_end[(int64_t)b * p.Lq + row[blk]]);
            } else {
                my_e[blk] = my_s[blk];
            }
        }
        if (my_e[blk] <= my_s[blk]) { my_s[blk] = BIG; my_e[blk] = 0; }
        lo = min(lo, my_s[blk]);
        hi = max(hi, my_e[blk]);
        in_lo = max(in_lo, my_s[blk]);
        in_hi = min(in_hi, my_e[blk]);
    }

    // work-group key range: [lo, hi) covers every non-empty row; tiles inside
    // [in_lo, in_hi) are visible to every row and need no masking
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
    // the same in every lane of the work-group: keep them in scalar registers
    lo = __builtin_amdgcn_readfirstlane(lo);
    hi = __builtin_amdgcn_readfirstlane(hi);
    in_lo = __builtin_amdgcn_readfirstlane(in_lo);
    in_hi = __builtin_amdgcn_readfirstlane(in_hi);

    // Q^T as B operand, resident for the whole kernel
    bf16x8 qreg[NBLK][8];
#pragma unroll
    for (int blk = 0; blk < NBLK; ++blk) {
        const uint16_t* qp = p.q + b * p.qs.b + h * p.qs.h + (int64_t)row[blk] * p.qs.s + g * 8;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) qreg[blk][kk] = as_bf16x8(ldg16(qp + kk * 16, row_ok[blk]));
    }

    const char* kbase = reinterpret_cast<const char*>(p.k + b * p.ks.b + hk * p.ks.h);
    const char* vbase = reinterpret_cast<const char*>(p.v + b * p.vs.b + hk * p.vs.h);
    const uint32_t krow_b = (uint32_t)p.ks.s * 2u, vrow_b = (uint32_t)p.vs.s * 2u;   // bytes per key row

    // global -> LDS: wave w moves the 1 KiB chunks w, w+4, w+8, w+12 (4 rows each)
    // of the K tile and of the V tile; lane i fills position i & 15 of row i >> 4.
    const int wave_u = wave;
    const int ld_r = lane >> 4;
    const uint32_t ld_c = (uint32_t)((lane & 15) ^ ((ld_r << 2) | wave_u)) * 16u;   // chunk this lane fetches
    const uint32_t lds0 = (uint32_t)(uintptr_t)&kv_lds[0][0][0];
    auto issue = [&](int kv0, int buf) {
        const char* kb = kbase + (int64_t)kv0 * krow_b;
        const char* vb = vbase + (int64_t)kv0 * vrow_b;
        const uint32_t slot = lds0 + (uint32_t)buf * (2 * TILE_BYTES) + (uint32_t)wave_u * 1024u;
        const int last = kv_hi - 1 - kv0;          // rows past `last` repeat it
        int lr = ld_r + 4 * wave_u;                // (a fresh copy: see the tile loop)
        asm volatile("" : "+v"(lr));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t r = (uint32_t)min(lr + 16 * j, last);
            dma16(kb, r * krow_b + ld_c, slot + j * 4096);
            dma16(vb, r * vrow_b + ld_c, slot + TILE_BYTES + j * 4096);
        }
    };

    // LDS -> operands.  K rows (A of S^T): 16 bytes at row * 256 + ((2 kk + g) ^ f(row)) * 16.
    const int f_row = ((l32 & 3) << 2) | ((l32 >> 2) & 3);
    const uint32_t k_rd = (uint32_t)(l32 * 256), k_h = (uint32_t)((g ^ f_row) << 4);
    // V^T (A of O^T += V^T P^T), keys in accumulator order: first half rows 16 j + 4 g + r,
    // second half 8 rows further down, whose f differs in bit 1.
    uint32_t v_rd[4][2];
    {
        const int r = (lane & 15) >> 2, t = lane & 3, u = (lane >> 4) & 1;
        const int low = (2 * u + (t >> 1)) ^ g;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
            v_rd[dt][0] = (uint32_t)((4 * g + r) * 256 + (4 * (dt ^ r) + low) * 16 + (t & 1) * 8);
            v_rd[dt][1] = (uint32_t)((4 * g + r + 8) * 256 + (4 * (dt ^ r) + (low ^ 2)) * 16 + (t & 1) * 8);
        }
    }

    // The same addresses as absolute LDS byte addresses for buffer 0.  The swizzles only touch address
    // bits that nothing else sets, so the address of k-step kk (K) or d tile dt (V) is the first one
    // with kk * 32 or dt * 64 XORed in: three registers serve the plain tile code and the
    // hand-scheduled loop (which wants all sixteen spelled out) alike.
    const uint32_t kaddr0 = lds0 + k_rd + k_h;
    const uint32_t vaddr0 = lds0 + TILE_BYTES + v_rd[0][0], vaddr1 = lds0 + TILE_BYTES + v_rd[0][1];
    const char* const lds_base = &kv_lds[0][0][0] - lds0;     // LDS byte address -> pointer

    f32x16 acc[NBLK][4];
    float m_i[NBLK], l_i[NBLK];
#pragma unroll
    for (int blk = 0; blk < NBLK; ++blk) {
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[blk][dt][v] = 0.f;
        m_i[blk] = -INFINITY;
        l_i[blk] = 0.f;
    }
    const float c = p.scale_log2e;
    const float cc = BIAS ? 1.f : c;              // factor from the carried scores to log2 units
    const float* brow = nullptr;                  // this lane's row of the bias
    if (BIAS) brow = p.bias + b * p.bias_b + h * p.bias_h + (int64_t)min(row[0], p.row_end - 1) * p.bias_r;

    const int t_begin = (hi > lo) ? lo / BN : 0;
    const int t_end = (hi > lo) ? (hi + BN - 1) / BN : 0;

    // the run [ta, ta + n_fast) of full tiles no row masks: an odd number of at least three
    int ta = t_begin, n_fast = 0;
    if (krow_b == vrow_b) {
        const int fa = max(t_begin, (in_lo + BN - 1) / BN);
        const int fb = min(t_end, min(in_hi, kv_hi) / BN);
        if (fb - fa >= 3) { ta = fa; n_fast = (fb - fa - 1) | 1; }
    }

    for (int phase = 0; phase < 3; ++phase) {
        if (phase == 1) {
            if (n_fast == 0) continue;
            int trips = n_fast >> 1;
            const char* kp = kbase + (int64_t)(ta * BN) * krow_b;
            const char* vp = vbase + (int64_t)(ta * BN) * vrow_b;
            uint32_t doff[4], kaddr[8], vaddr[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) doff[j] = (uint32_t)(4 * (wave_u + 4 * j) + ld_r) * krow_b + ld_c;
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) kaddr[kk] = kaddr0 ^ (uint32_t)(kk * 32);
#pragma unroll
            for (int dt = 0; dt < 4; ++dt) {
                vaddr[2 * dt] = vaddr0 ^ (uint32_t)(dt * 64);
                vaddr[2 * dt + 1] = vaddr1 ^ (uint32_t)(dt * 64);
            }
            const uint32_t lds_w = lds0 + (uint32_t)wave_u * 1024u;
            if constexpr (NBLK == 1) {
                asm volatile(
#include "lvx_fwd_loop_bf16.inc"
                    : "+{v[0:15]}"(acc[0][0]), "+{v[16:31]}"(acc[0][1]), "+{v[32:47]}"(acc[0][2]), "+{v[48:63]}"(acc[0][3]),
                      "+{v244}"(m_i[0]), "+{v245}"(l_i[0]), "+{s[44:45]}"(kp), "+{s[46:47]}"(vp), "+{s51}"(trips)
                    : "{v[64:67]}"(qreg[0][0]), "{v[68:71]}"(qreg[0][1]), "{v[72:75]}"(qreg[0][2]), "{v[76:79]}"(qreg[0][3]),
                      "{v[80:83]}"(qreg[0][4]), "{v[84:87]}"(qreg[0][5]), "{v[88:91]}"(qreg[0][6]), "{v[92:95]}"(qreg[0][7]),
                      "{v224}"(kaddr[0]), "{v225}"(kaddr[1]), "{v226}"(kaddr[2]), "{v227}"(kaddr[3]),
                      "{v228}"(kaddr[4]), "{v229}"(kaddr[5]), "{v230}"(kaddr[6]), "{v231}"(kaddr[7]),
                      "{v232}"(vaddr[0]), "{v233}"(vaddr[1]), "{v234}"(vaddr[2]), "{v235}"(vaddr[3]),
                      "{v236}"(vaddr[4]), "{v237}"(vaddr[5]), "{v238}"(vaddr[6]), "{v239}"(vaddr[7]),
                      "{v240}"(doff[0]), "{v241}"(doff[1]), "{v242}"(doff[2]), "{v243}"(doff[3]),
                      "{s40}"(cc), "{s41}"(-INFINITY), "{s42}"(RESCALE_LOG2), "{s48}"((uint32_t)BN * krow_b),
                      "{s49}"((uint32_t)BN * vrow_b), "{s50}"(lds_w)
                    : "memory", "vcc", "scc", "m0", "s52", "s53", "s54", "s55", "s56", LVX_FWD_LOOP_CLOBBERS);
            } else {
                // O^T and Q^T travel in VGPRs; the statement parks them in accumulation registers while it
                // runs and hands them back in the registers they came in
                asm volatile(
#include "lvx_fwd_loop_wide.inc"
                    : "+{v[0:15]}"(acc[0][0]), "+{v[16:31]}"(acc[0][1]), "+{v[32:47]}"(acc[0][2]), "+{v[48:63]}"(acc[0][3]),
                      "+{v[64:79]}"(acc[NBLK - 1][0]), "+{v[80:95]}"(acc[NBLK - 1][1]), "+{v[96:111]}"(acc[NBLK - 1][2]),
                      "+{v[112:127]}"(acc[NBLK - 1][3]),
                      "+{v[128:131]}"(qreg[0][0]), "+{v[132:135]}"(qreg[0][1]), "+{v[136:139]}"(qreg[0][2]), "+{v[140:143]}"(qreg[0][3]),
                      "+{v[144:147]}"(qreg[0][4]), "+{v[148:151]}"(qreg[0][5]), "+{v[152:155]}"(qreg[0][6]), "+{v[156:159]}"(qreg[0][7]),
                      "+{v[160:163]}"(qreg[NBLK - 1][0]), "+{v[164:167]}"(qreg[NBLK - 1][1]), "+{v[168:171]}"(qreg[NBLK - 1][2]),
                      "+{v[172:175]}"(qreg[NBLK - 1][3]), "+{v[176:179]}"(qreg[NBLK - 1][4]), "+{v[180:183]}"(qreg[NBLK - 1][5]),
                      "+{v[184:187]}"(qreg[NBLK - 1][6]), "+{v[188:191]}"(qreg[NBLK - 1][7]),
                      "+{v220}"(m_i[0]), "+{v221}"(m_i[NBLK - 1]), "+{v222}"(l_i[0]), "+{v223}"(l_i[NBLK - 1]),
                      "+{s[44:45]}"(kp), "+{s[46:47]}"(vp), "+{s51}"(trips)
                    : "{v200}"(kaddr[0]), "{v201}"(kaddr[1]), "{v202}"(kaddr[2]), "{v203}"(kaddr[3]),
                      "{v204}"(kaddr[4]), "{v205}"(kaddr[5]), "{v206}"(kaddr[6]), "{v207}"(kaddr[7]),
                      "{v208}"(vaddr[0]), "{v209}"(vaddr[1]), "{v210}"(vaddr[2]), "{v211}"(vaddr[3]),
                      "{v212}"(vaddr[4]), "{v213}"(vaddr[5]), "{v214}"(vaddr[6]), "{v215}"(vaddr[7]),
                      "{v216}"(doff[0]), "{v217}"(doff[1]), "{v218}"(doff[2]), "{v219}"(doff[3]),
                      "{s40}"(cc), "{s41}"(-INFINITY), "{s42}"(RESCALE_LOG2), "{s48}"((uint32_t)BN * krow_b),
                      "{s49}"((uint32_t)BN * vrow_b), "{s50}"(lds_w)
                    : "memory", "vcc", "scc", "m0", "s52", "s53", "s54", "s55", "s56", "s58", "s59", "s60", "s61",
                      LVX_FWD_WIDE_CLOBBERS);
            }
            continue;
        }
        const int t0 = phase == 0 ? t_begin : ta + n_fast;
        const int t1 = phase == 0 ? ta : t_end;
        if (t1 <= t0) continue;
        __syncthreads();     // the tile buffers are free: every wave is done with the previous phase
        issue(t0 * BN, 0);
        for (int t = t0; t < t1; ++t) {
            const int kv0 = t * BN;
            const int buf = (t - t0) & 1;
            // fresh copies the compiler cannot hoist: the sixteen derived addresses are then formed
            // tile by tile (an XOR each) instead of being kept - and spilled - across the whole loop
            uint32_t ka0 = kaddr0, va0 = vaddr0, va1 = vaddr1;
            asm volatile("" : "+v"(ka0), "+v"(va0), "+v"(va1));

            // tile t has landed (this wave's part: vmcnt; everyone's: barrier); the
            // barrier also says every wave is done reading tile t-1, whose buffer
            // the loads of tile t+1 may now overwrite
            wait_vmcnt<0>();
            __syncthreads();
            if (t + 1 < t1) issue(kv0 + BN, buf ^ 1);

            // S^T = K Q^T : rows = keys (two 32-key sub-tiles), cols = text rows.
            // All 16 K operands are requested before the first MFMA, so the LDS
            // latency is paid once per tile and not once per k-step.
            bf16x8 ka[8][2];
    #pragma unroll
            for (int kk = 0; kk < 8; ++kk) {
                const char* kp = lds_base + (ka0 ^ (uint32_t)(kk * 32)) + buf * (2 * TILE_BYTES);
                ka[kk][0] = *reinterpret_cast<const bf16x8*>(kp);
                ka[kk][1] = *reinterpret_cast<const bf16x8*>(kp + 32 * 256);
            }
            __builtin_amdgcn_sched_barrier(0);
            f32x16 s0[NBLK], s1[NBLK];
    #pragma unroll
            for (int blk = 0; blk < NBLK; ++blk) {
    #pragma unroll
                for (int v = 0; v < 16; ++v) { s0[blk][v] = 0.f; s1[blk][v] = 0.f; }
    #pragma unroll
                for (int kk = 0; kk < 8; ++kk) {
                    s0[blk] = E::mfma(ka[kk][0], qreg[blk][kk], s0[blk]);
                    s1[blk] = E::mfma(ka[kk][1], qreg[blk][kk], s1[blk]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            // V^T operands of this tile: requested now, they land during the softmax
            u32x2 va[4][4][2];
    #pragma unroll
            for (int dt = 0; dt < 4; ++dt)
    #pragma unroll
                for (int j = 0; j < 4; ++j) {
                    va[dt][j][0] = lds_read_tr16(reinterpret_cast<const uint16_t*>(lds_base + (va0 ^ (uint32_t)(dt * 64)) + buf * (2 * TILE_BYTES) + j * 4096));
                    va[dt][j][1] = lds_read_tr16(reinterpret_cast<const uint16_t*>(lds_base + (va1 ^ (uint32_t)(dt * 64)) + buf * (2 * TILE_BYTES) + j * 4096));
                }
            __builtin_amdgcn_sched_barrier(0);

    #pragma unroll
            for (int blk = 0; blk < NBLK; ++blk) {
                if (kv0 < in_lo || kv0 + BN > in_hi) {
    #pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int kv = kv0 + acc_row(v, g);
                        if (kv < my_s[blk] || kv >= my_e[blk]) s0[blk][v] = -INFINITY;
                        if (kv + 32 < my_s[blk] || kv + 32 >= my_e[blk]) s1[blk][v] = -INFINITY;
                    }
                }

                float mx = max3(s0[blk][0], s1[blk][0], s0[blk][1]);
                mx = max3(mx, s1[blk][1], s0[blk][2]);
    #pragma unroll
                for (int v = 3; v < 16; v += 1) mx = max3(mx, s1[blk][v - 1], s0[blk][v]);
                mx = fmaxf(mx, s1[blk][15]);
                {   // other half of the wave holds the other 32 keys of the same text row
                    const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
                    mx = max3(__uint_as_float(sw[0]), __uint_as_float(sw[1]), m_i[blk]);
                }
                // Lazy rescale: the reference point m_i of a row only moves when the row
                // maximum has grown by more than 2^RESCALE_LOG2 since it was set, so P may
                // reach 2^RESCALE_LOG2 instead of 1 (harmless in fp32 / bf16) and the
                // rescale of O happens a few times per row instead of almost every tile.
                const float mcand = mx * cc;                      // mx >= m_i
                const float m_ic = m_i[blk] * cc;
                const bool move = (mx != -INFINITY) && !(mcand - m_ic <= RESCALE_LOG2);
                const float alpha = move ? __builtin_amdgcn_exp2f(m_ic - mcand) : 1.f;
                if (move) m_i[blk] = mx;
                const float mc = (m_i[blk] == -INFINITY) ? 0.f : m_i[blk] * cc;

                // P^T as B operand: k-step j covers keys 16j..16j+15 of the tile.  The row
                // sum is taken in fp32 before the rounding to bf16 (summing the rounded
                // values would put the LSE off by up to a bf16 ulp of the largest term).
                bf16x8 pb[4];
                float rs0 = 0.f, rs1 = 0.f;
    #pragma unroll
                for (int j = 0; j < 2; ++j) {
                    u32x4 u0, u1;
    #pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int v = 8 * j + 2 * e;
                        const float a0 = __builtin_amdgcn_exp2f(fmaf(s0[blk][v], cc, -mc)), a1 = __builtin_amdgcn_exp2f(fmaf(s0[blk][v + 1], cc, -mc));
                        const float b0 = __builtin_amdgcn_exp2f(fmaf(s1[blk][v], cc, -mc)), b1 = __builtin_amdgcn_exp2f(fmaf(s1[blk][v + 1], cc, -mc));
                        rs0 += a0 + a1;
                        rs1 += b0 + b1;
                        u0[e] = E::pack(a0, a1);
                        u1[e] = E::pack(b0, b1);
                    }
                    pb[j] = as_bf16x8(u0);
                    pb[2 + j] = as_bf16x8(u1);
                }
                l_i[blk] = l_i[blk] * alpha + (rs0 + rs1);

                if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {   // the running max moved for some row
    #pragma unroll
                    for (int dt = 0; dt < 4; ++dt)
    #pragma unroll
                        for (int v = 0; v < 16; ++v) acc[blk][dt][v] *= alpha;
                }

                // O^T += V^T P^T
                __builtin_amdgcn_sched_barrier(0);
    #pragma unroll
                for (int dt = 0; dt < 4; ++dt)
    #pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const u32x4 a = {va[dt][j][0][0], va[dt][j][0][1], va[dt][j][1][0], va[dt][j][1][1]};
                        acc[blk][dt] = E::mfma(as_bf16x8(a), pb[j], acc[blk][dt]);
                    }
            }
        }
    }

    // epilogue: the two lane halves hold partial row sums of the same row
#pragma unroll
    for (int blk = 0; blk < NBLK; ++blk) {
        const float l_tot = l_i[blk] + __shfl_xor(l_i[blk], 32);
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        if (row_ok[blk]) {
            uint16_t* op = p.o + split * p.o_split_stride + b * p.os.b + h * p.os.h + (int64_t)row[blk] * p.os.s;
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                for (int vg = 0; vg < 4; ++vg) {
                    u32x2 w;
                    w[0] = E::pack(acc[blk][dt][4 * vg] * inv, acc[blk][dt][4 * vg + 1] * inv);
                    w[1] = E::pack(acc[blk][dt][4 * vg + 2] * inv, acc[blk][dt][4 * vg + 3] * inv);
                    *reinterpret_cast<u32x2*>(op + dt * 32 + 8 * vg + 4 * g) = w;
                }
            if (g == 0) {
                const float lse = l_tot > 0.f ? m_i[blk] * (BIAS ? LN2_F : p.scale) + __logf(l_tot) : -INFINITY;
                p.lse[split * p.lse_split_stride + ((int64_t)b * p.Hq + h) * p.lse_bh_stride + row[blk]] = lse;
            }
        }
    }
}

}  // namespace

namespace {
template <int DH, bool F16>
hipError_t launch_fwd_t(const FwdParams& p, bool masked, hipStream_t st) {
    const int grid = ((p.total_wg + 7) / 8) * 8;
    if (p.bias) {
        if (masked) return launch1((fwd_kernel<DH, true, true, F16>), dim3(grid), dim3(256), st, p);
        else return launch1((fwd_kernel<DH, false, true, F16>), dim3(grid), dim3(256), st, p);
    } else if (DH == 128 && !F16 && !masked) {
        // (with an interval mask the plain kernel is the faster one: the edges of the rows' intervals leave
        // the hand-scheduled loop short runs, and its register needs cost the tile code around it)
        if (p.wide) return launch1((fwd_kernel_pipe<2>), dim3(grid), dim3(256), st, p);
        return launch1((fwd_kernel_pipe<1>), dim3(grid), dim3(256), st, p);
    } else {
        if (masked) return launch1((fwd_kernel<DH, true, false, F16>), dim3(grid), dim3(256), st, p);
        else return launch1((fwd_kernel<DH, false, false, F16>), dim3(grid), dim3(256), st, p);
    }
}
}  // namespace

hipError_t launch_fwd(const FwdParams& p, bool masked, hipStream_t st) {
    switch (p.D) {
        case 16: return p.f16 ? launch_fwd_t<16, true>(p, masked, st) : launch_fwd_t<16, false>(p, masked, st);
        case 32: return p.f16 ? launch_fwd_t<32, true>(p, masked, st) : launch_fwd_t<32, false>(p, masked, st);
        case 64: return p.f16 ? launch_fwd_t<64, true>(p, masked, st) : launch_fwd_t<64, false>(p, masked, st);
        case 128: return p.f16 ? launch_fwd_t<128, true>(p, masked, st) : launch_fwd_t<128, false>(p, masked, st);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace lvx
