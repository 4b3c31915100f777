// Internal launch interface between the C-ABI layer (lvx_api.hip) and the
// kernel translation units.  All sizes have been validated by the caller.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lvx {

// Queues kernel(p) and returns that launch's own error code.  The thread's sticky "last error"
// (which may hold an unrelated component's earlier failure) is neither read nor cleared.
template <typename P>
inline hipError_t launch1(void (*kernel)(P), dim3 grid, dim3 block, hipStream_t st, const P& p) {
    P arg = p;
    void* args[] = {&arg};
    return hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, args, 0, st);
}

struct Strides3 {
    int64_t b, h, s;
};

struct FwdParams {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    uint16_t* o;
    float* lse;
    Strides3 qs, ks, vs, os;
    int64_t o_split_stride;    // elements between the partial O of two key splits
    int64_t lse_split_stride;  // floats between the partial LSE of two key splits
    int64_t lse_bh_stride;     // floats between two (b, h) rows of LSE
    const int32_t* kv_len;
    const int32_t* kv_start;
    const int32_t* kv_end;
    const float* bias;         // dense additive bias or nullptr; element strides below
    int64_t bias_b, bias_h, bias_r;
    int B, Hq, Hkv, Lq, Lkv;
    int D;                     // head dimension: 16, 32, 64 or 128
    int G;                     // q heads per kv head
    int HG;                    // q heads a work-group covers (one per wave)
    int RS;                    // row sub-tiles a work-group covers per head
    int wide;                  // 1: a wave owns 64 rows (two blocks of 32) instead of 32; bf16 without bias only
    int row_begin, row_end;
    int n_row_tiles, n_head_groups, nsplit, split_len, total_wg;
    float scale, scale_log2e;
    int f16;                   // element type of q, k, v, o: 0 bf16, 1 fp16
};

struct MergeParams {
    uint16_t* o_acc;
    float* l_acc;
    const uint16_t* o_part;
    const float* l_part;
    Strides3 oa, op;
    int64_t o_part_stride;     // elements between consecutive partials
    int64_t l_part_stride;     // floats between consecutive partials
    int64_t l_acc_bh, l_part_bh;
    int nparts;
    int use_acc;               // 1: fold into the existing accumulator, 0: overwrite
    // with use_acc and several parts: where the accumulator is read from when it is not
    // (o_acc, l_acc) itself, which then only receive the result (null: in place)
    const uint16_t* o_in;
    const float* l_in;
    Strides3 oi;
    int64_t l_in_bh;
    int B, Hq, Lq, row_begin, row_end;
    int f16;
    int D;                     // head dimension: 16, 32, 64 or 128 (0 reads as 128)
};

// Per text row the hull of the keys a dense bias leaves visible (entries other than -inf).
struct BiasHullParams {
    const float* bias;
    int64_t bias_b, bias_h, bias_r;
    int32_t* kv_start;         // [B, Lq]: written by the hull kernel, read by the interval test
    int32_t* kv_end;           // [B, Lq]
    int B, heads, Lq, Lkv;     // heads: 1 (bias broadcast over heads) or Hq
    int32_t* flag;             // interval test only: set to 1 when the bias is not 0 everywhere inside the hull
};
hipError_t launch_bias_hull(const BiasHullParams& p, hipStream_t st);
hipError_t launch_bias_interval(const BiasHullParams& p, hipStream_t st);

struct PreParams {
    const uint16_t* o;
    const uint16_t* dout;
    float* delta;
    Strides3 os, ds;
    int B, Hq, Lq, row_begin, row_end;
    int f16;
    int D;                     // head dimension: 16, 32, 64 or 128 (0 reads as 128)
};

struct BwdParams {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    const uint16_t* dout;
    const float* meta;         // per (b, h, 32-row tile): 32 x LSE*log2(e) (+inf for dead rows), 32 x delta*scale
    uint16_t* ds_ws;           // dS^T workspace [B*Hq][token blocks][row tiles][128 tokens][32 rows]
    int64_t ws_ld;             // elements per token block (row tiles * 4096)
    int64_t ws_bh;             // elements per (b, h) slab
    void* dk;
    void* dv;
    Strides3 qs, ks, vs, dos, dks, dvs;
    const int32_t* kv_len;
    const int32_t* kv_start;
    const int32_t* kv_end;
    const float* bias;         // dense additive bias or nullptr; element strides below
    int64_t bias_b, bias_h, bias_r;
    int B, Hq, Hkv, Lq, Lkv, G;
    int D;                     // head dimension: 16, 32, 64 or 128
    int row_begin, row_end;
    int n_kv_blocks;
    int n_blocks;              // token blocks of all (b, kv head): B * Hkv * n_kv_blocks
    int blocks_per_xcd;        // ceil(n_blocks / 8): the token blocks an XCD's work-groups take
    int whole_blocks;          // of an XCD's blocks, the first so many get one work-group each (0 .. blocks_per_xcd),
    int mid_blocks, q_splits;  // the next mid_blocks are shared by q_splits work-groups each, every one taking a range of steps,
    int q_splits2;             // and the others by q_splits2 (>= 1) work-groups each
    int dkv_mode;              // 0: store 16-bit, 1: fp32 +=, 2: fp32 atomic += (q_splits > 1: the shared blocks)
    // mode 2: where and how the work-group of a block it owns alone writes (whole_mode 0 or 1)
    void* dk_whole;
    void* dv_whole;
    Strides3 dks_whole, dvs_whole;
    int whole_mode;
    float scale, scale_log2e;
    // Interval masks: the 32-row tiles each token block has to visit (the others see none of
    // its tokens) as up to 4 runs of consecutive tiles, live_runs[(b * n_kv_blocks + block) * 8
    // + 2 i + {0, 1}] = first tile and number of tiles of run i (0 tiles: unused).  Null: every tile.
    const int32_t* live_runs;
    int f16;                   // element type of q, k, v, dout, the dS^T workspace and (mode 0) dk, dv
};

// Which (token block, 32-row tile) pairs an interval mask leaves alive, at the granularity the
// dQ GEMM needs: rows are taken in groups of `group` tiles (one M tile of that GEMM); a group's
// hull is the smallest range of whole token blocks that holds every key some row of the group
// sees, and all tiles of a group are alive for exactly the blocks of its hull.
struct LiveParams {
    const int32_t* kv_len;     // may be null
    const int32_t* kv_start;
    const int32_t* kv_end;
    int32_t* hull;             // out: [B][n_groups][2] token range (multiples of 128), (0, 0) if empty
    int32_t* live_runs;        // out, see BwdParams; a fifth run and later ones are merged into the
                               // fourth together with the gaps between them (visiting more is harmless)
    int32_t* order;            // out (may be null): the B * n_groups group indices b * n_groups + grp,
                               // longest hull first (ties in index order)
    int B, Lq, Lkv, row_begin, row_end, n_tiles, group, n_groups, n_kv_blocks;
};
hipError_t launch_bwd_live(const LiveParams& p, hipStream_t st);

// Row metadata of the backward in the form its kernel consumes, one 256-byte
// record per (b, h, 32-row tile of the window).
struct MetaParams {
    const float* lse;
    const float* delta;
    float* out;
    int B, Hq, Lq, row_begin, row_end, n_tiles;
    float scale;
    // up to two regions the same launch zero-fills (the fp32 scratches the call accumulates
    // into); dst 16-byte aligned, n16 = number of 16-byte chunks, 0: none
    uint32_t* zero_dst[2];
    int64_t zero_n16[2];
    int meta_blocks;           // filled by the launcher: blocks [0, meta_blocks) write records
};


struct CastParams {
    const float* src;
    uint16_t* dst;
    Strides3 ds;
    // a second tensor of the same sizes, cast by the same launch (null: none)
    const float* src2;
    uint16_t* dst2;
    Strides3 ds2;
    // the fp32 dK / dV scratch of the backward, (H, L) = (tokens, kv heads): rows of token blocks that
    // the kernel wrote directly (the first skip_whole of every skip_bpx blocks of the list (b, kv
    // head, block), skip_nkvb blocks per (b, kv head), skip_nblocks in all) are left alone.  skip_bpx 0: none.
    int skip_bpx, skip_whole, skip_nkvb, skip_nblocks;
    int B, H, L;
    int transposed;   // 0: src is [B*H][L][D]; 1: src is [B*H][D][L]
    int nsum;         // transposed only: the result is the sum of nsum such sources (0 or 1: one),
    int64_t sum_stride;   // sum_stride floats apart
    int f16;          // destination type: 0 bf16, 1 fp16
    int D;            // head dimension: 16, 32, 64 or 128 (0 reads as 128)
};

// One GEMM problem C[M,N] = sum over segments A_s[M,K_s] * B_s[K_s,N].
struct GemmProblem {
    const uint16_t* A[2];
    const uint16_t* Bm[2];
    int64_t lda[2], ldb[2];
    int K[2];
    int nseg;
    uint16_t* C;
    int64_t ldc;
};

// `nprob` problems of one shape, each repeated over `nbatch` batch entries.
// Batch entry z = zo * batch_inner + zi addresses
//   A + z * a_batch,  B + zo * b_outer + (zi / b_group) * b_inner,
//   C + zo * c_outer + zi * c_inner
// and, when k_len is given, contracts over only the first k_len[zo] values of k.
struct GemmParams {
    GemmProblem prob[2];
    int nprob;
    int M, N;
    int M_ld;                  // rows of A that may be loaded (>= M; rows in [M, M_ld) are padding)
    int tiles_m, tiles_n, total_wg;   // filled in by launch_gemm for the tile it picks
    int nbatch, batch_inner, b_group;
    int64_t a_batch, b_outer, b_inner, c_outer, c_inner;
    const int32_t* k_len;
    // RMS norm over each aligned group of 128 columns of problem 0's C (the k_norm of the K
    // projection), applied to the accumulator before the store: y = bf16(w * bf16(x * r)),
    // r = rsqrt(mean(x^2) + eps), x = the bf16-rounded product.  norm_w: 128 bf16 weights
    // (null: off).  c_raw (optional): x itself, indexed like C.  rstd (optional):
    // r[m * (N / 128) + n / 128].
    const uint16_t* norm_w;
    float norm_eps;
    uint16_t* c_raw;
    float* rstd;
    // Per (outer batch index, M tile) contraction range of segment 0: k_range[(zo * tiles_m +
    // tm) * 2 + {0, 1}] = first and one-past-last k (multiples of 128); null: all of K[0].
    const int32_t* k_range;
    // With k_range (one problem, no split contraction): the (outer batch index, M tile) pairs
    // zo * tiles_m + tm in the order the work-groups are to take them, longest range first
    // (null: in index order).
    const int32_t* m_order;
    int f16;                   // element type of A, B, C (and the norm weight): 0 bf16, 1 fp16
    // Split contraction (single-segment problems): k_splits work-groups per C tile, each
    // contracting k_split_len values of k (a multiple of 128) and storing its partial tile
    // in fp32 to its own slice of the TRANSPOSED scratch
    // c32[split * c32_split + z * c32_batch + n * c32_ld + m] (the accumulator holds C^T, so
    // a wave's lanes then write consecutive addresses; every split writes its whole tile,
    // zeros if its range is empty) instead of storing bf16 to C; the caller sums the slices.
    // k_splits <= 1: off.
    int k_splits, k_split_len;
    float* c32;
    int64_t c32_split, c32_batch;
    int c32_ld;
    // a_tiled_m > 0: A (stored [K][M]) is cut into contiguous [128 k][32 m] tiles,
    // a_tiled_m of them per block of 128 k; lda is ignored
    int a_tiled_m;
};

hipError_t launch_fwd(const FwdParams& p, bool masked, hipStream_t st);   // p.bias selects the bias variant
hipError_t launch_merge(const MergeParams& p, hipStream_t st);
hipError_t launch_preprocess(const PreParams& p, hipStream_t st);
hipError_t launch_bwd(const BwdParams& p, bool masked, hipStream_t st);
hipError_t launch_cast(const CastParams& p, hipStream_t st);
hipError_t launch_bwd_meta(const MetaParams& p, hipStream_t st);

// Backward of the 128-wide RMS norm: rows of dy, x [M][heads][128] (row strides ldy, ldx), r [M][heads].
struct NormBwdParams {
    const uint16_t* dy;
    const uint16_t* x;
    const float* rstd;
    const uint16_t* w;
    uint16_t* dx;
    float* dw;        // [128] fp32, added to (null: not wanted)
    int64_t ldy, ldx, lddx;
    int M, heads;
    int f16;
};
hipError_t launch_norm_bwd(const NormBwdParams& p, hipStream_t st);
// a_mcontig: A is stored [K][M] (m contiguous); b_ncontig: B is stored [K][N].
hipError_t launch_gemm(const GemmParams& p, bool a_mcontig, bool b_ncontig, hipStream_t st);

}  // namespace lvx
