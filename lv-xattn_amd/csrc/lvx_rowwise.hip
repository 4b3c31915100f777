// The HBM-bound row-wise kernels of the path: the LSE rescale-merge, the
// backward preprocess (delta = rowsum(O * dO)) and the final fp32 -> bf16
// rounding of an accumulator.  With head_dim 128 a row is 16 lanes x 16 bytes,
// so a 256-thread group streams 16 rows per pass with fully coalesced 256-byte
// row segments; with head_dim 64 / 32 / 16 it is 8 / 4 / 2 lanes and 32 / 64 / 128 rows per pass.
#include "lvx_common.hpp"
#include "lvx_kernels.hpp"

#include <algorithm>
#include <climits>

namespace lvx {

namespace {

constexpr int MAX_PARTS = 16;

// log2 of the 16-byte chunks (lanes) per row
__device__ __forceinline__ int chunk_shift(int head_dim) {
    return head_dim == 64 ? 3 : head_dim == 32 ? 2 : head_dim == 16 ? 1 : 4;
}

template <class E>
__device__ __forceinline__ void unpack8(u32x4 u, float f[8]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        f[2 * j] = E::lo(u[j]);
        f[2 * j + 1] = E::hi(u[j]);
    }
}

// (o_acc, l_acc) <- merge(acc?, part_0 .. part_{n-1}) for every (b, h, row).
template <bool F16>
__global__ __launch_bounds__(256) void merge_kernel(const MergeParams p) {
    using E = Elt<F16>;
    const int nrows = p.row_end - p.row_begin;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int sh = chunk_shift(p.D);
    const int chunk = (int)(idx & ((1 << sh) - 1));
    const int64_t r = idx >> sh;
    if (r >= (int64_t)p.B * p.Hq * nrows) return;
    const int row = p.row_begin + (int)(r % nrows);
    const int bh = (int)(r / nrows);
    const int b = bh / p.Hq, h = bh % p.Hq;

    float la = -INFINITY;
    if (p.use_acc) la = p.l_in ? p.l_in[(int64_t)bh * p.l_in_bh + row] : p.l_acc[(int64_t)bh * p.l_acc_bh + row];
    float lp[MAX_PARTS];
    float m = la;
#pragma unroll
    for (int i = 0; i < MAX_PARTS; ++i) {
        if (i < p.nparts) {
            lp[i] = p.l_part[i * p.l_part_stride + (int64_t)bh * p.l_part_bh + row];
            m = fmaxf(m, lp[i]);
        }
    }
    const float ms = (m == -INFINITY) ? 0.f : m;
    float wa = __expf(la - ms);
    float den = wa;
#pragma unroll
    for (int i = 0; i < MAX_PARTS; ++i) {
        if (i < p.nparts) {
            lp[i] = __expf(lp[i] - ms);
            den += lp[i];
        }
    }
    const float inv = den > 0.f ? 1.f / den : 0.f;

    float out[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) out[j] = 0.f;
    uint16_t* oa = p.o_acc + b * p.oa.b + h * p.oa.h + (int64_t)row * p.oa.s + chunk * 8;
    if (p.use_acc) {
        float f[8];
        const uint16_t* oin = p.o_in ? p.o_in + b * p.oi.b + h * p.oi.h + (int64_t)row * p.oi.s + chunk * 8 : oa;
        unpack8<E>(*reinterpret_cast<const u32x4*>(oin), f);
        const float w = wa * inv;
        // an accumulator with weight 0 (L = -inf: nothing folded in yet) may hold anything
        if (w > 0.f) {
#pragma unroll
            for (int j = 0; j < 8; ++j) out[j] = f[j] * w;
        }
    }
    const uint16_t* op = p.o_part + b * p.op.b + h * p.op.h + (int64_t)row * p.op.s + chunk * 8;
#pragma unroll
    for (int i = 0; i < MAX_PARTS; ++i) {
        if (i < p.nparts) {
            float f[8];
            unpack8<E>(*reinterpret_cast<const u32x4*>(op + i * p.o_part_stride), f);
            const float w = lp[i] * inv;
            // a part with weight 0 may hold anything (it saw no key)
            if (w > 0.f) {
#pragma unroll
                for (int j = 0; j < 8; ++j) out[j] = fmaf(f[j], w, out[j]);
            }
        }
    }
    u32x4 u;
#pragma unroll
    for (int j = 0; j < 4; ++j) u[j] = E::pack(out[2 * j], out[2 * j + 1]);
    *reinterpret_cast<u32x4*>(oa) = u;
    if (chunk == 0) p.l_acc[(int64_t)bh * p.l_acc_bh + row] = den > 0.f ? ms + __logf(den) : -INFINITY;
}

// The same for one part folded into the accumulator (what lvx_merge does every round), two rows
// per thread: every load of both rows is issued before the first use, so a thread keeps
// 64 + 8 bytes in flight.  780 bytes per (row, head).
template <bool F16>
__global__ __launch_bounds__(256) void merge_pair_kernel(const MergeParams p) {
    using E = Elt<F16>;
    const int nrows = p.row_end - p.row_begin;
    const int64_t total = (int64_t)p.B * p.Hq * nrows;
    const int64_t half = (total + 1) / 2;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int sh = chunk_shift(p.D);
    const int chunk = (int)(idx & ((1 << sh) - 1));
    const int64_t r0 = idx >> sh;
    if (r0 >= half) return;
    int64_t rr[2] = {r0, r0 + half};
    const bool ok1 = rr[1] < total;
    if (!ok1) rr[1] = r0;
    uint16_t* oa[2];
    const uint16_t* op[2];
    float* la_p[2];
    float la[2], lb[2];
    u32x4 ua[2], ub[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int row = p.row_begin + (int)(rr[k] % nrows);
        const int bh = (int)(rr[k] / nrows);
        const int b = bh / p.Hq, h = bh % p.Hq;
        oa[k] = p.o_acc + b * p.oa.b + h * p.oa.h + (int64_t)row * p.oa.s + chunk * 8;
        op[k] = p.o_part + b * p.op.b + h * p.op.h + (int64_t)row * p.op.s + chunk * 8;
        la_p[k] = p.l_acc + (int64_t)bh * p.l_acc_bh + row;
        la[k] = *la_p[k];
        lb[k] = p.l_part[(int64_t)bh * p.l_part_bh + row];
        ua[k] = *reinterpret_cast<const u32x4*>(oa[k]);
        ub[k] = *reinterpret_cast<const u32x4*>(op[k]);
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        if (k == 1 && !ok1) break;
        const float m = fmaxf(la[k], lb[k]);
        const float ms = (m == -INFINITY) ? 0.f : m;
        const float wa = __expf(la[k] - ms), wb = __expf(lb[k] - ms);
        const float den = wa + wb;
        const float inv = den > 0.f ? 1.f / den : 0.f;
        // a side with weight 0 may hold anything (it saw no key, or nothing was folded in yet)
        const float ca = wa * inv, cb = wb * inv;
        float fa[8], fb[8];
        unpack8<E>(ua[k], fa);
        unpack8<E>(ub[k], fb);
        u32x4 u;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float x0 = (ca > 0.f ? fa[2 * j] * ca : 0.f) + (cb > 0.f ? fb[2 * j] * cb : 0.f);
            const float x1 = (ca > 0.f ? fa[2 * j + 1] * ca : 0.f) + (cb > 0.f ? fb[2 * j + 1] * cb : 0.f);
            u[j] = E::pack(x0, x1);
        }
        *reinterpret_cast<u32x4*>(oa[k]) = u;
        if (chunk == 0) *la_p[k] = den > 0.f ? ms + __logf(den) : -INFINITY;
    }
}

// delta = rowsum(O * dO): head_dim / 8 lanes x 16 bytes per row and tensor, two rows per thread with all
// four loads issued before the first use.  516 bytes per (row, head).
template <bool F16>
__global__ __launch_bounds__(256) void preprocess_kernel(const PreParams p) {
    using E = Elt<F16>;
    const int nrows = p.row_end - p.row_begin;
    const int64_t total = (int64_t)p.B * p.Hq * nrows;
    const int64_t half = (total + 1) / 2;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int sh = chunk_shift(p.D);
    const int chunk = (int)(idx & ((1 << sh) - 1));
    const int64_t r0 = idx >> sh;
    const bool ok0 = r0 < half;                         // the lanes of a row share the flags
    const bool ok1 = ok0 && r0 + half < total;
    const int64_t rr[2] = {ok0 ? r0 : 0, ok1 ? r0 + half : 0};
    u32x4 uo[2], ud[2];
    float* out[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int row = p.row_begin + (int)(rr[k] % nrows);
        const int bh = (int)(rr[k] / nrows);
        const int b = bh / p.Hq, h = bh % p.Hq;
        const bool ok = k ? ok1 : ok0;
        uo[k] = ldg16(p.o + b * p.os.b + h * p.os.h + (int64_t)row * p.os.s + chunk * 8, ok);
        ud[k] = ldg16(p.dout + b * p.ds.b + h * p.ds.h + (int64_t)row * p.ds.s + chunk * 8, ok);
        out[k] = p.delta + (int64_t)bh * p.Lq + row;
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        float fo[8], fd[8];
        unpack8<E>(uo[k], fo);
        unpack8<E>(ud[k], fd);
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) s = fmaf(fo[j], fd[j], s);
        if (sh >= 4) s += __shfl_xor(s, 8);
        if (sh >= 3) s += __shfl_xor(s, 4);
        if (sh >= 2) s += __shfl_xor(s, 2);
        s += __shfl_xor(s, 1);
        if ((k ? ok1 : ok0) && chunk == 0) *out[k] = s;
    }
}

// LSE and delta of the window, re-expressed once for the backward kernel: the
// exponent offset LSE * log2(e), +inf for rows that saw no key or lie past the
// window (so that P = exp2(x - inf) = 0 there), and delta * scale (0 past the
// window), grouped per 32-row tile so that one 256-byte load fetches a tile's lot.
__global__ __launch_bounds__(256) void bwd_meta_kernel(const MetaParams p) {
    // the other blocks of the launch zero the scratches (stores rather than hipMemsetAsync, so
    // that callers may capture the stream)
    if ((int)blockIdx.x >= p.meta_blocks) {
        const u32x4 z = {0u, 0u, 0u, 0u};
        const int64_t first = (int64_t)(blockIdx.x - p.meta_blocks) * 256 + threadIdx.x;
        const int64_t stride = (int64_t)(gridDim.x - p.meta_blocks) * 256;
#pragma unroll
        for (int r = 0; r < 2; ++r)
            for (int64_t i = first; i < p.zero_n16[r]; i += stride) reinterpret_cast<u32x4*>(p.zero_dst[r])[i] = z;
        return;
    }
    const int rows_pad = p.n_tiles * 32;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)p.B * p.Hq * rows_pad) return;
    const int r = (int)(idx % rows_pad);
    const int64_t bh = idx / rows_pad;
    const int row = p.row_begin + r;
    const bool ok = row < p.row_end;
    const float l = ok ? p.lse[bh * p.Lq + row] : -INFINITY;
    const float d = ok ? p.delta[bh * p.Lq + row] : 0.f;
    float* o = p.out + (bh * p.n_tiles + (r >> 5)) * 64 + (r & 31);
    o[0] = (l == -INFINITY) ? INFINITY : l * 1.4426950408889634f;
    o[32] = d * p.scale;
}

// One wave per (b, text row): first and one-past-last key whose bias is not -inf, over all heads
// the bias distinguishes.  An empty row gets (0, 0).
__global__ __launch_bounds__(256) void bias_hull_kernel(const BiasHullParams p) {
    const int64_t rw = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (rw >= (int64_t)p.B * p.Lq) return;
    const int b = (int)(rw / p.Lq), row = (int)(rw % p.Lq);
    int lo = INT_MAX, hi = 0;
    for (int h = 0; h < p.heads; ++h) {
        const float* br = p.bias + b * p.bias_b + h * p.bias_h + (int64_t)row * p.bias_r;
        for (int k0 = 4 * lane; k0 < p.Lkv; k0 += 256) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(br + k0);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (k0 + j < p.Lkv && !(v[j] == -INFINITY)) { lo = min(lo, k0 + j); hi = max(hi, k0 + j + 1); }
        }
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        lo = min(lo, __shfl_xor(lo, o));
        hi = max(hi, __shfl_xor(hi, o));
    }
    if (lane == 0) {
        p.kv_start[rw] = hi > 0 ? lo : 0;
        p.kv_end[rw] = hi;
    }
}

// One wave per (b, text row): sets *p.flag when an entry of the row's bias inside [kv_start, kv_end)
// is not exactly zero, i.e. when the bias is more than the interval mask its hull describes.
__global__ __launch_bounds__(256) void bias_interval_kernel(const BiasHullParams p) {
    const int64_t rw = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (rw >= (int64_t)p.B * p.Lq) return;
    const int b = (int)(rw / p.Lq), row = (int)(rw % p.Lq);
    const int lo = max(p.kv_start[rw], 0), hi = min(p.kv_end[rw], p.Lkv);
    bool other = false;
    for (int h = 0; h < p.heads; ++h) {
        const float* br = p.bias + b * p.bias_b + h * p.bias_h + (int64_t)row * p.bias_r;
        for (int k0 = (lo & ~3) + 4 * lane; k0 < hi; k0 += 256) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(br + k0);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (k0 + j >= lo && k0 + j < hi && !(v[j] == 0.f)) other = true;
        }
    }
    if (__builtin_amdgcn_ballot_w64(other) != 0 && lane == 0) atomicOr(p.flag, 1);
}

// One wave per (group of row tiles, b): the hull of the rows' key intervals in whole token blocks.
__global__ __launch_bounds__(64) void bwd_hull_kernel(const LiveParams p) {
    const int grp = blockIdx.x, b = blockIdx.y, lane = threadIdx.x;
    const int r0 = p.row_begin + grp * p.group * 32;
    const int r1 = min(r0 + p.group * 32, p.row_end);
    const int kv_len = p.kv_len ? min(p.kv_len[b], p.Lkv) : p.Lkv;
    int lo = INT_MAX, hi = 0;
    for (int r = r0 + lane; r < r1; r += 64) {
        const int s = max(p.kv_start[(int64_t)b * p.Lq + r], 0);
        const int e = min(p.kv_end[(int64_t)b * p.Lq + r], kv_len);
        if (e > s) { lo = min(lo, s); hi = max(hi, e); }
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        lo = min(lo, __shfl_xor(lo, o));
        hi = max(hi, __shfl_xor(hi, o));
    }
    if (lane == 0) {
        int32_t* h = p.hull + ((int64_t)b * p.n_groups + grp) * 2;
        h[0] = hi > 0 ? (lo / 128) * 128 : 0;
        h[1] = (hi + 127) / 128 * 128;
    }
}

// One thread per (token block, b): the runs of consecutive row tiles whose group's hull holds the block.
// Blocks past those (b == 0 only) rank the groups by hull length, one thread per group.
__global__ __launch_bounds__(64) void bwd_live_kernel(const LiveParams p) {
    const int live_blocks = (p.n_kv_blocks + 63) / 64;
    if ((int)blockIdx.x >= live_blocks) {
        const int n = p.B * p.n_groups;
        const int i = ((int)blockIdx.x - live_blocks) * 64 + threadIdx.x;
        if (blockIdx.y != 0 || i >= n) return;
        const int len = p.hull[2 * i + 1] - p.hull[2 * i];
        int rank = 0;
        for (int j = 0; j < n; ++j) {
            const int lj = p.hull[2 * j + 1] - p.hull[2 * j];
            rank += (lj > len || (lj == len && j < i)) ? 1 : 0;
        }
        p.order[rank] = i;
        return;
    }
    const int kblk = blockIdx.x * 64 + threadIdx.x, b = blockIdx.y;
    if (kblk >= p.n_kv_blocks) return;
    const int kvb = kblk * 128;
    int32_t* out = p.live_runs + ((int64_t)b * p.n_kv_blocks + kblk) * 8;
    int nr = 0, start = 0;
    bool open = false;
    for (int grp = 0; grp < p.n_groups; ++grp) {
        const int32_t* h = p.hull + ((int64_t)b * p.n_groups + grp) * 2;
        const bool live = h[0] <= kvb && kvb < h[1];
        const int t0 = grp * p.group, t1 = min(t0 + p.group, p.n_tiles);
        if (live) {
            if (!open && nr < 4) { start = t0; ++nr; }
            out[2 * (nr - 1)] = start;
            out[2 * (nr - 1) + 1] = t1 - start;
        }
        open = live;
    }
    for (int i = nr; i < 4; ++i) { out[2 * i] = 0; out[2 * i + 1] = 0; }
}

template <bool F16>
__global__ __launch_bounds__(256) void cast_kernel(const CastParams p) {
    using E = Elt<F16>;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int sh = chunk_shift(p.D);
    const int Dh = 8 << sh;
    const int chunk = (int)(idx & ((1 << sh) - 1));
    const int64_t r = idx >> sh;
    if (r >= (int64_t)p.B * p.H * p.L) return;
    const int row = (int)(r % p.L);
    const int bh = (int)(r / p.L);
    const int b = bh / p.H, h = bh % p.H;
    if (p.skip_bpx) {      // h is a token, row a kv head
        const int blk = (h >> 7) + p.skip_nkvb * (b + p.B * row);
        const int first = blk / p.skip_bpx * p.skip_bpx;
        if (blk - first < min(p.skip_whole, p.skip_nblocks - first)) return;
    }
    const bool second = blockIdx.y != 0;
    const f32x4* s = reinterpret_cast<const f32x4*>((second ? p.src2 : p.src) + r * Dh + chunk * 8);
    const f32x4 a = s[0], c = s[1];
    u32x4 u;
    u[0] = E::pack(a[0], a[1]);
    u[1] = E::pack(a[2], a[3]);
    u[2] = E::pack(c[0], c[1]);
    u[3] = E::pack(c[2], c[3]);
    const Strides3 ds = second ? p.ds2 : p.ds;
    *reinterpret_cast<u32x4*>((second ? p.dst2 : p.dst) + b * ds.b + h * ds.h + (int64_t)row * ds.s + chunk * 8) = u;
}

// Same from a transposed source [B*H][D][L], or the sum of several: adjacent threads take
// adjacent rows, so the eight strided reads of a thread are coalesced across the wave.
template <bool F16>
__global__ __launch_bounds__(256) void cast_t_kernel(const CastParams p) {
    using E = Elt<F16>;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int sh = chunk_shift(p.D);
    const int Dh = 8 << sh;
    if (idx >= ((int64_t)p.B * p.H * p.L << sh)) return;
    const int row = (int)(idx % p.L);
    const int chunk = (int)((idx / p.L) & ((1 << sh) - 1));
    const int bh = (int)(idx / ((int64_t)p.L << sh));
    const int b = bh / p.H, h = bh % p.H;
    const float* s = p.src + ((int64_t)bh * Dh + chunk * 8) * p.L + row;
    float a[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) a[j] = s[(int64_t)j * p.L];
    for (int k = 1; k < p.nsum; ++k) {
        s += p.sum_stride;
#pragma unroll
        for (int j = 0; j < 8; ++j) a[j] += s[(int64_t)j * p.L];
    }
    u32x4 u;
#pragma unroll
    for (int j = 0; j < 4; ++j) u[j] = E::pack(a[2 * j], a[2 * j + 1]);
    *reinterpret_cast<u32x4*>(p.dst + b * p.ds.b + h * p.ds.h + (int64_t)row * p.ds.s + chunk * 8) = u;
}

// Backward of y = w * bf16(x * r) over 128-wide rows: with xh = x * r and gg = dy * w,
//   dx = r * (gg - xh * mean(gg * xh)),   dw += sum over rows of dy * bf16(xh).
// 16 lanes per row (8 columns each); a thread keeps the dw partial sums of its 8 columns
// over the rows it visits, the block folds them through LDS and adds them with atomics.
template <bool F16>
__global__ __launch_bounds__(256) void norm_bwd_kernel(const NormBwdParams p) {
    using E = Elt<F16>;
    __shared__ float fold[16][16][8];
    const int sub = threadIdx.x & 15, grp = threadIdx.x >> 4;
    const int64_t nrows = (int64_t)p.M * p.heads;
    const u32x4 wu = *reinterpret_cast<const u32x4*>(p.w + sub * 8);
    float w[8], dwp[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) { w[2 * j] = E::lo(wu[j]); w[2 * j + 1] = E::hi(wu[j]); }
#pragma unroll
    for (int j = 0; j < 8; ++j) dwp[j] = 0.f;
    for (int64_t row = (int64_t)blockIdx.x * 16 + grp; row < nrows; row += (int64_t)gridDim.x * 16) {
        const int64_t m = row / p.heads;
        const int h = (int)(row % p.heads);
        const u32x4 du = *reinterpret_cast<const u32x4*>(p.dy + m * p.ldy + h * 128 + sub * 8);
        const u32x4 xu = *reinterpret_cast<const u32x4*>(p.x + m * p.ldx + h * 128 + sub * 8);
        const float r = p.rstd[row];
        float gg[8], xh[8], c = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float d0 = E::lo(du[j]), d1 = E::hi(du[j]);
            xh[2 * j] = E::lo(xu[j]) * r;
            xh[2 * j + 1] = E::hi(xu[j]) * r;
            gg[2 * j] = d0 * w[2 * j];
            gg[2 * j + 1] = d1 * w[2 * j + 1];
            const uint32_t xb = E::pack(xh[2 * j], xh[2 * j + 1]);
            dwp[2 * j] = fmaf(d0, E::lo(xb), dwp[2 * j]);
            dwp[2 * j + 1] = fmaf(d1, E::hi(xb), dwp[2 * j + 1]);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) c = fmaf(gg[j], xh[j], c);
#pragma unroll
        for (int o = 1; o < 16; o <<= 1) c += __shfl_xor(c, o);
        c *= 1.f / 128.f;
        u32x4 out;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            out[j] = E::pack(r * (gg[2 * j] - xh[2 * j] * c), r * (gg[2 * j + 1] - xh[2 * j + 1] * c));
        *reinterpret_cast<u32x4*>(p.dx + m * p.lddx + h * 128 + sub * 8) = out;
    }
    if (!p.dw) return;
#pragma unroll
    for (int j = 0; j < 8; ++j) fold[grp][sub][j] = dwp[j];
    __syncthreads();
    if (threadIdx.x < 128) {
        const int s2 = threadIdx.x >> 3, j = threadIdx.x & 7;
        float t = 0.f;
#pragma unroll
        for (int gi = 0; gi < 16; ++gi) t += fold[gi][s2][j];
        unsafeAtomicAdd(p.dw + threadIdx.x, t);
    }
}

inline int blocks_for(int64_t rows) { return (int)((rows * 16 + 255) / 256); }

}  // namespace

hipError_t launch_merge(const MergeParams& p, hipStream_t st) {
    const int64_t rows = (int64_t)p.B * p.Hq * (p.row_end - p.row_begin);
    if (rows == 0) return hipSuccess;
    if (p.nparts == 1 && p.use_acc && !p.o_in) {
        const dim3 grid(blocks_for((rows + 1) / 2));
        if (p.f16) return launch1(merge_pair_kernel<true>, grid, dim3(256), st, p);
        return launch1(merge_pair_kernel<false>, grid, dim3(256), st, p);
    }
    if (p.f16) return launch1(merge_kernel<true>, dim3(blocks_for(rows)), dim3(256), st, p);
    else return launch1(merge_kernel<false>, dim3(blocks_for(rows)), dim3(256), st, p);
}

hipError_t launch_preprocess(const PreParams& p, hipStream_t st) {
    const int64_t rows = (int64_t)p.B * p.Hq * (p.row_end - p.row_begin);
    if (rows == 0) return hipSuccess;
    if (p.f16) return launch1(preprocess_kernel<true>, dim3(blocks_for((rows + 1) / 2)), dim3(256), st, p);
    else return launch1(preprocess_kernel<false>, dim3(blocks_for((rows + 1) / 2)), dim3(256), st, p);
}

hipError_t launch_bwd_meta(const MetaParams& p0, hipStream_t st) {
    MetaParams p = p0;
    const int64_t n = (int64_t)p.B * p.Hq * p.n_tiles * 32;
    const int64_t z = p.zero_n16[0] + p.zero_n16[1];
    if (n == 0 && z == 0) return hipSuccess;
    p.meta_blocks = (int)((n + 255) / 256);
    const int zero_blocks = (int)std::min<int64_t>((z + 255) / 256, 2048);
    return launch1(bwd_meta_kernel, dim3((unsigned)(p.meta_blocks + zero_blocks)), dim3(256), st, p);
}

hipError_t launch_bwd_live(const LiveParams& p, hipStream_t st) {
    if (p.B <= 0 || p.n_groups <= 0 || p.n_kv_blocks <= 0) return hipSuccess;
    const hipError_t e = launch1(bwd_hull_kernel, dim3(p.n_groups, p.B), dim3(64), st, p);
    if (e != hipSuccess) return e;
    const int rank_blocks = p.order ? (p.B * p.n_groups + 63) / 64 : 0;
    return launch1(bwd_live_kernel, dim3((p.n_kv_blocks + 63) / 64 + rank_blocks, p.B), dim3(64), st, p);
}

hipError_t launch_bias_hull(const BiasHullParams& p, hipStream_t st) {
    const int64_t rows = (int64_t)p.B * p.Lq;
    if (rows == 0) return hipSuccess;
    return launch1(bias_hull_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), st, p);
}

hipError_t launch_bias_interval(const BiasHullParams& p, hipStream_t st) {
    const int64_t rows = (int64_t)p.B * p.Lq;
    if (rows == 0) return hipSuccess;
    return launch1(bias_interval_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), st, p);
}

hipError_t launch_norm_bwd(const NormBwdParams& p, hipStream_t st) {
    const int64_t rows = (int64_t)p.M * p.heads;
    if (rows == 0) return hipSuccess;
    const int grid = (int)std::min<int64_t>((rows + 15) / 16, 2048);
    if (p.f16) return launch1(norm_bwd_kernel<true>, dim3(grid), dim3(256), st, p);
    else return launch1(norm_bwd_kernel<false>, dim3(grid), dim3(256), st, p);
}

hipError_t launch_cast(const CastParams& p, hipStream_t st) {
    const int64_t rows = (int64_t)p.B * p.H * p.L;
    if (rows == 0) return hipSuccess;
    const dim3 grid(blocks_for(rows), !p.transposed && p.src2 ? 2 : 1);
    if (p.transposed) {
        if (p.src2) return hipErrorInvalidValue;
        if (p.f16) return launch1(cast_t_kernel<true>, grid, dim3(256), st, p);
        else return launch1(cast_t_kernel<false>, grid, dim3(256), st, p);
    } else {
        if (p.f16) return launch1(cast_kernel<true>, grid, dim3(256), st, p);
        else return launch1(cast_kernel<false>, grid, dim3(256), st, p);
    }
}

}  // namespace lvx
