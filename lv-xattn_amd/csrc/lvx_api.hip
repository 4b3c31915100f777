// C-ABI layer: argument validation on the host (nothing is launched when a
// check fails), translation to the internal launch parameters, error strings.
#include "../../include/lvx.h"
#include "lvx_kernels.hpp"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <mutex>

using namespace lvx;

namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_tensor(const lvx_tensor* t) {
    if (!t || !t->ptr) return LVX_ERR_NULL;
    if (!aligned16(t->ptr)) return LVX_ERR_ALIGN;
    if ((t->stride_b % 8) || (t->stride_h % 8) || (t->stride_s % 8)) return LVX_ERR_ALIGN;
    if (t->stride_s <= 0) return LVX_ERR_SHAPE;
    return LVX_OK;
}

int check_shape(const lvx_attn_shape* s) {
    if (!s) return LVX_ERR_NULL;
    if (s->dtype != LVX_BF16 && s->dtype != LVX_F16) return LVX_ERR_DTYPE;
    if (s->D != 128 && s->D != 64 && s->D != 32 && s->D != 16) return LVX_ERR_HEAD_DIM;
    if (s->B <= 0 || s->Hq <= 0 || s->Hkv <= 0 || s->Lq <= 0 || s->Lkv <= 0) return LVX_ERR_SHAPE;
    if (s->Hq % s->Hkv) return LVX_ERR_SHAPE;
    if (!(s->scale > 0.f) || !std::isfinite(s->scale)) return LVX_ERR_SCALE;
    if ((s->kv_start == nullptr) != (s->kv_end == nullptr)) return LVX_ERR_NULL;
    if (s->bias) {
        // rows are read in groups of 4 keys with 16-byte loads: every row must start on a
        // 16-byte boundary and be readable up to Lkv rounded up to 4
        if (reinterpret_cast<uintptr_t>(s->bias) & 15) return LVX_ERR_ALIGN;
        if ((s->bias_stride_r | s->bias_stride_h | s->bias_stride_b) & 3) return LVX_ERR_ALIGN;
        if (s->bias_stride_r < (s->Lkv + 3) / 4 * 4) return LVX_ERR_SHAPE;
    }
    return LVX_OK;
}

int check_rows(const lvx_attn_shape* s, int32_t row_begin, int32_t row_count) {
    if (row_begin < 0 || row_count < 0 || (int64_t)row_begin + row_count > s->Lq) return LVX_ERR_SHAPE;
    return LVX_OK;
}

inline Strides3 st3(const lvx_tensor* t) { return Strides3{t->stride_b, t->stride_h, t->stride_s}; }

inline int gcd(int a, int b) { return b ? gcd(b, a % b) : a; }

constexpr float LOG2E = 1.4426950408889634f;
constexpr int FWD_BN = 64;
constexpr int MAX_SPLITS = 16;

#define LVX_TRY(expr)            \
    do {                         \
        int rc_ = (expr);        \
        if (rc_ != LVX_OK) return rc_; \
    } while (0)

}  // namespace

static void fill_grid(GemmParams& g, int M, int N, int nprob, int nbatch);

// Device memory of lvx_fwd_noalloc: the key-split partials live in this file-scope array
// instead of a caller's workspace.  Every GPU the library runs on holds its own copy at its
// own address until the process ends; the address is asked for once per device.
constexpr size_t NOALLOC_SCRATCH_BYTES = LVX_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
constexpr int MAX_RANKED_GROUPS = 1024;    // 256-row groups of a masked backward that are still ranked by length
std::mutex scratch_mutex;
void* scratch_ptr[MAX_DEVICES];      // per device: where that device keeps `scratch`

// The device address of `scratch` on the current device (the array's name is a host-side
// stand-in, not an address a kernel can use).
int scratch_on_current_device(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return static_cast<int>(e);
    if (dev < 0 || dev >= MAX_DEVICES) return LVX_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return static_cast<int>(e);
        if (!ptr) return LVX_ERR_UNSUPPORTED;
        scratch_ptr[dev] = ptr;
    }
    *out = scratch_ptr[dev];
    return LVX_OK;
}
}  // namespace

extern "C" {

int lvx_version(void) { return LVX_VERSION; }

const char* lvx_strerror(int code) {
    switch (code) {
        case LVX_OK: return "ok";
        case LVX_ERR_NULL: return "a required pointer is NULL";
        case LVX_ERR_ALIGN: return "pointer not 16-byte aligned or stride not a multiple of 8 elements";
        case LVX_ERR_SHAPE: return "bad sizes or row window";
        case LVX_ERR_HEAD_DIM: return "head_dim must be 16, 32, 64 or 128";
        case LVX_ERR_DTYPE: return "dtype must be LVX_BF16 or LVX_F16";
        case LVX_ERR_SCALE: return "scale must be finite and > 0";
        case LVX_ERR_WORKSPACE: return "workspace missing or too small";
        case LVX_ERR_UNSUPPORTED: return "not supported by this build";
        default: break;
    }
    if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
    return "unknown lvx error";
}

size_t lvx_fwd_workspace_bytes(const lvx_attn_shape* s, int32_t row_count, int32_t kv_splits) {
    if (!s || kv_splits <= 1 || row_count <= 0) return 0;
    const size_t rows = (size_t)s->B * s->Hq * row_count;
    return (size_t)kv_splits * rows * (s->D * sizeof(uint16_t) + sizeof(float));
}

static int cu_count();

// Whether the forward runs in its wide form (a wave owns 64 rows and its SIMD; one work-group per
// CU): bf16, head_dim 128, without a dense bias or an interval mask, whole 64-row blocks, and enough work-groups
// that every CU has one.
static bool fwd_wide(const lvx_attn_shape* s, int32_t row_count, int rs, int kv_splits) {
    if (s->dtype != LVX_BF16 || s->D != 128 || s->bias || s->kv_start) return false;
    if (const char* e = getenv("LVX_FWD_WIDE")) return atoi(e) != 0;
    if (row_count % (64 * rs) != 0) return false;
    const int64_t wgs = (int64_t)s->B * (s->Hq / (4 / rs)) * (row_count / (64 * rs)) * kv_splits;
    return wgs >= cu_count();
}

// lvx_fwd, and lvx_fwd_acc when (o_in, l_in) is given: the result is then merged with that
// incoming accumulator before it is written to (o, lse).
static int fwd_impl(const lvx_attn_shape* s, const lvx_tensor* q, const lvx_tensor* k, const lvx_tensor* v,
                    const lvx_tensor* o, float* lse, int32_t row_begin, int32_t row_count, int32_t kv_splits,
                    void* workspace, size_t workspace_bytes, void* stream, const lvx_tensor* o_in, const float* l_in) {
    LVX_TRY(check_shape(s));
    LVX_TRY(check_tensor(q));
    LVX_TRY(check_tensor(k));
    LVX_TRY(check_tensor(v));
    LVX_TRY(check_tensor(o));
    if (!lse) return LVX_ERR_NULL;
    LVX_TRY(check_rows(s, row_begin, row_count));
    if (kv_splits < 1 || kv_splits > MAX_SPLITS) return LVX_ERR_SHAPE;
    if (row_count == 0) return LVX_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);

    FwdParams p{};
    p.f16 = s->dtype == LVX_F16;
    p.D = s->D;
    p.q = static_cast<const uint16_t*>(q->ptr);
    p.k = static_cast<const uint16_t*>(k->ptr);
    p.v = static_cast<const uint16_t*>(v->ptr);
    p.qs = st3(q); p.ks = st3(k); p.vs = st3(v);
    p.kv_len = s->kv_len; p.kv_start = s->kv_start; p.kv_end = s->kv_end;
    p.bias = s->bias; p.bias_b = s->bias_stride_b; p.bias_h = s->bias_stride_h; p.bias_r = s->bias_stride_r;
    p.B = s->B; p.Hq = s->Hq; p.Hkv = s->Hkv; p.Lq = s->Lq; p.Lkv = s->Lkv;
    p.G = s->Hq / s->Hkv;
    p.HG = gcd(p.G, 4);
    p.RS = 4 / p.HG;
    p.row_begin = row_begin; p.row_end = row_begin + row_count;
    p.wide = fwd_wide(s, row_count, p.RS, kv_splits) ? 1 : 0;
    const int wg_rows = (p.wide ? 64 : 32) * p.RS;
    p.n_row_tiles = (row_count + wg_rows - 1) / wg_rows;
    p.n_head_groups = s->Hq / p.HG;
    p.scale = s->scale; p.scale_log2e = s->scale * LOG2E;

    int nsplit = kv_splits;
    int split_len = ((s->Lkv + nsplit - 1) / nsplit + FWD_BN - 1) / FWD_BN * FWD_BN;
    nsplit = (s->Lkv + split_len - 1) / split_len;
    p.nsplit = nsplit;
    p.split_len = split_len;
    p.total_wg = s->B * p.n_head_groups * nsplit * p.n_row_tiles;

    if (nsplit == 1) {
        p.o = static_cast<uint16_t*>(o->ptr);
        p.os = st3(o);
        p.lse = lse;
        p.lse_bh_stride = s->Lq;
        const hipError_t e1 = launch_fwd(p, s->kv_start != nullptr, st);
        if (e1 != hipSuccess || !o_in) return static_cast<int>(e1);
        // one partial, written straight to (o, lse): fold the incoming accumulator into it (the
        // merge is symmetric, so which side is "the accumulator" does not matter)
        MergeParams m{};
        m.f16 = s->dtype == LVX_F16;
        m.D = s->D;
        m.o_acc = static_cast<uint16_t*>(o->ptr);
        m.l_acc = lse;
        m.o_part = static_cast<const uint16_t*>(o_in->ptr);
        m.l_part = l_in;
        m.oa = st3(o);
        m.op = st3(o_in);
        m.l_acc_bh = s->Lq;
        m.l_part_bh = s->Lq;
        m.nparts = 1;
        m.use_acc = 1;
        m.B = s->B; m.Hq = s->Hq; m.Lq = s->Lq;
        m.row_begin = row_begin; m.row_end = row_begin + row_count;
        return static_cast<int>(launch_merge(m, st));
    }

    // key splits: partials [split][B*Hq][row_count][D] + LSE [split][B*Hq][row_count]
    const size_t need = lvx_fwd_workspace_bytes(s, row_count, nsplit);
    if (!workspace || workspace_bytes < need) return LVX_ERR_WORKSPACE;
    if (!aligned16(workspace)) return LVX_ERR_ALIGN;
    const int64_t rows = (int64_t)s->B * s->Hq * row_count;
    uint16_t* o_ws = static_cast<uint16_t*>(workspace);
    float* l_ws = reinterpret_cast<float*>(o_ws + (int64_t)nsplit * rows * s->D);
    // the kernel indexes partials by absolute row: bias the bases by -row_begin
    p.o = o_ws - (int64_t)row_begin * s->D;
    p.os = Strides3{(int64_t)s->Hq * row_count * s->D, (int64_t)row_count * s->D, s->D};
    p.o_split_stride = rows * s->D;
    p.lse = l_ws - row_begin;
    p.lse_bh_stride = row_count;
    p.lse_split_stride = rows;
    hipError_t e = launch_fwd(p, s->kv_start != nullptr, st);
    if (e != hipSuccess) return static_cast<int>(e);

    MergeParams m{};
    m.f16 = s->dtype == LVX_F16;
    m.D = s->D;
    m.o_acc = static_cast<uint16_t*>(o->ptr);
    m.l_acc = lse;
    m.o_part = p.o;
    m.l_part = p.lse;
    m.oa = st3(o);
    m.op = p.os;
    m.o_part_stride = p.o_split_stride;
    m.l_part_stride = p.lse_split_stride;
    m.l_acc_bh = s->Lq;
    m.l_part_bh = row_count;
    m.nparts = nsplit;
    m.use_acc = 0;
    if (o_in) {      // the partials and the incoming accumulator in one launch
        m.use_acc = 1;
        m.o_in = static_cast<const uint16_t*>(o_in->ptr);
        m.l_in = l_in;
        m.oi = st3(o_in);
        m.l_in_bh = s->Lq;
    }
    m.B = s->B; m.Hq = s->Hq; m.Lq = s->Lq;
    m.row_begin = row_begin; m.row_end = row_begin + row_count;
    return static_cast<int>(launch_merge(m, st));
}

int lvx_fwd(const lvx_attn_shape* s, const lvx_tensor* q, const lvx_tensor* k, const lvx_tensor* v,
            const lvx_tensor* o, float* lse, int32_t row_begin, int32_t row_count, int32_t kv_splits,
            void* workspace, size_t workspace_bytes, void* stream) {
    return fwd_impl(s, q, k, v, o, lse, row_begin, row_count, kv_splits, workspace, workspace_bytes, stream,
                    nullptr, nullptr);
}

int lvx_fwd_acc(const lvx_attn_shape* s, const lvx_tensor* q, const lvx_tensor* k, const lvx_tensor* v,
                const lvx_tensor* o_in, const float* l_in, const lvx_tensor* o, float* lse, int32_t row_begin,
                int32_t row_count, int32_t kv_splits, void* workspace, size_t workspace_bytes, void* stream) {
    if (!o_in) return LVX_ERR_NULL;
    LVX_TRY(check_tensor(o_in));
    if (!l_in) return LVX_ERR_NULL;
    // the result is formed out of place: the kernel writes (o, lse) of the window before the merge
    // reads (o_in, l_in), so the row windows of the two may not share memory
    if (o && o_in->ptr == o->ptr) return LVX_ERR_SHAPE;
    if (l_in == lse) return LVX_ERR_SHAPE;
    if (o && o->ptr && s && row_count > 0 && s->B > 0 && s->Hq > 0) {
        auto span = [&](const lvx_tensor* t, const char*& lo, const char*& hi) {
            const int64_t last = (int64_t)(s->B - 1) * t->stride_b + (int64_t)(s->Hq - 1) * t->stride_h +
                                 (int64_t)(row_begin + row_count - 1) * t->stride_s + s->D;
            lo = static_cast<const char*>(t->ptr) + (int64_t)row_begin * t->stride_s * 2;
            hi = static_cast<const char*>(t->ptr) + last * 2;
        };
        const char *alo, *ahi, *blo, *bhi;
        span(o, alo, ahi);
        span(o_in, blo, bhi);
        if (alo < bhi && blo < ahi) return LVX_ERR_SHAPE;
    }
    if (lse && l_in && s && row_count > 0) {
        const int64_t rows = (int64_t)s->B * s->Hq * s->Lq;
        if (l_in < lse + rows && lse < l_in + rows) return LVX_ERR_SHAPE;
    }
    return fwd_impl(s, q, k, v, o, lse, row_begin, row_count, kv_splits, workspace, workspace_bytes, stream,
                    o_in, l_in);
}

size_t lvx_noalloc_scratch_bytes(void) { return NOALLOC_SCRATCH_BYTES; }

int lvx_fwd_noalloc(const lvx_attn_shape* s, const lvx_tensor* q, const lvx_tensor* k, const lvx_tensor* v,
                    const lvx_tensor* o, float* lse, int32_t row_begin, int32_t row_count, int32_t kv_splits,
                    void* stream) {
    // argument errors first, as lvx_fwd reports them
    LVX_TRY(check_shape(s));
    if (kv_splits < 1 || kv_splits > MAX_SPLITS) return LVX_ERR_SHAPE;
    if (row_count > 0 && lvx_fwd_workspace_bytes(s, row_count, kv_splits) > NOALLOC_SCRATCH_BYTES)
        return LVX_ERR_WORKSPACE;     // the partials of this call do not fit the library's own array
    void* ws = nullptr;
    LVX_TRY(scratch_on_current_device(&ws));
    return lvx_fwd(s, q, k, v, o, lse, row_begin, row_count, kv_splits, ws, NOALLOC_SCRATCH_BYTES, stream);
}

int lvx_merge(const lvx_attn_shape* s, const lvx_tensor* o_acc, float* l_acc, const lvx_tensor* o_part,
              const float* l_part, int32_t row_begin, int32_t row_count, void* stream) {
    LVX_TRY(check_shape(s));
    LVX_TRY(check_tensor(o_acc));
    LVX_TRY(check_tensor(o_part));
    if (!l_acc || !l_part) return LVX_ERR_NULL;
    LVX_TRY(check_rows(s, row_begin, row_count));
    MergeParams m{};
    m.f16 = s->dtype == LVX_F16;
    m.D = s->D;
    m.o_acc = static_cast<uint16_t*>(o_acc->ptr);
    m.l_acc = l_acc;
    m.o_part = static_cast<const uint16_t*>(o_part->ptr);
    m.l_part = l_part;
    m.oa = st3(o_acc);
    m.op = st3(o_part);
    m.l_acc_bh = s->Lq;
    m.l_part_bh = s->Lq;
    m.nparts = 1;
    m.use_acc = 1;
    m.B = s->B; m.Hq = s->Hq; m.Lq = s->Lq;
    m.row_begin = row_begin; m.row_end = row_begin + row_count;
    return static_cast<int>(launch_merge(m, static_cast<hipStream_t>(stream)));
}

int lvx_bias_hull(const lvx_attn_shape* s, int32_t* kv_start, int32_t* kv_end, void* stream) {
    LVX_TRY(check_shape(s));
    if (!s->bias || !kv_start || !kv_end) return LVX_ERR_NULL;
    BiasHullParams p{};
    p.bias = s->bias; p.bias_b = s->bias_stride_b; p.bias_h = s->bias_stride_h; p.bias_r = s->bias_stride_r;
    p.kv_start = kv_start; p.kv_end = kv_end;
    p.B = s->B; p.heads = s->bias_stride_h ? s->Hq : 1; p.Lq = s->Lq; p.Lkv = s->Lkv;
    return static_cast<int>(launch_bias_hull(p, static_cast<hipStream_t>(stream)));
}

int lvx_bias_is_interval(const lvx_attn_shape* s, const int32_t* kv_start, const int32_t* kv_end, int32_t* not_interval,
                         void* stream) {
    LVX_TRY(check_shape(s));
    if (!s->bias || !kv_start || !kv_end || !not_interval) return LVX_ERR_NULL;
    BiasHullParams p{};
    p.bias = s->bias; p.bias_b = s->bias_stride_b; p.bias_h = s->bias_stride_h; p.bias_r = s->bias_stride_r;
    p.kv_start = const_cast<int32_t*>(kv_start); p.kv_end = const_cast<int32_t*>(kv_end);
    p.B = s->B; p.heads = s->bias_stride_h ? s->Hq : 1; p.Lq = s->Lq; p.Lkv = s->Lkv;
    p.flag = not_interval;
    return static_cast<int>(launch_bias_interval(p, static_cast<hipStream_t>(stream)));
}

int lvx_bwd_preprocess(const lvx_attn_shape* s, const lvx_tensor* o, const lvx_tensor* dout, float* delta,
                       int32_t row_begin, int32_t row_count, void* stream) {
    LVX_TRY(check_shape(s));
    LVX_TRY(check_tensor(o));
    LVX_TRY(check_tensor(dout));
    if (!delta) return LVX_ERR_NULL;
    LVX_TRY(check_rows(s, row_begin, row_count));
    PreParams p{};
    p.f16 = s->dtype == LVX_F16;
    p.D = s->D;
    p.o = static_cast<const uint16_t*>(o->ptr);
    p.dout = static_cast<const uint16_t*>(dout->ptr);
    p.delta = delta;
    p.os = st3(o); p.ds = st3(dout);
    p.B = s->B; p.Hq = s->Hq; p.Lq = s->Lq;
    p.row_begin = row_begin; p.row_end = row_begin + row_count;
    return static_cast<int>(launch_preprocess(p, static_cast<hipStream_t>(stream)));
}

// Work-groups of the backward are long (every step of a token block) and one
// fits a CU, so a grid that is not a multiple of the CU count wastes up to one
// whole round.  Splitting the steps of every token block over `S` work-groups
// (which then add their dK/dV with atomics into an fp32 scratch that is zeroed before
// and rounded after) evens that out.  S minimises
//     rounds(S) * (steps / S + WG_COST) + (S > 1 ? SPLIT_COST : 0)        [in steps]
// with ranges of at least 32 steps; WG_COST is what a work-group spends outside its
// steps (operand load, ring fill, epilogue: about 8 us = 6 steps), SPLIT_COST the zero-fill, the
// two casts and the slower atomic epilogue (about 70 us).  rounds(S) = ceil(blocks * S / CUs)
// for equal work-groups.  With an interval mask they differ in length (a token block
// visits only the row tiles that see it; half of them is assumed); given at least two per CU the
// dispatcher fills the tail by itself and rounds(S) is the plain quotient: splitting then
// rarely pays (cfg4: 0.98 ms with 5 splits, 0.86 ms with none).
// CUs of the device that is current (the one the caller's stream belongs to), asked for once per device
static int cu_count() {
    static int cached[MAX_DEVICES];          // 0: not asked yet
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return 256;
    int n = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        __atomic_store_n(&cached[dev], n, __ATOMIC_RELAXED);
    }
    return n;
}

// How the token blocks of a launch are handed to work-groups (see bwd_kernel): per XCD, the first
// `whole` blocks get one work-group each, the next `mid` blocks `splits` work-groups each and the
// others `splits2` each.
struct BwdCut {
    int blocks_per_xcd, whole, mid, splits, splits2;
    bool any_split() const { return (mid > 0 && splits > 1) || (whole + mid < blocks_per_xcd && splits2 > 1); }
};

static BwdCut choose_bwd_cut(int blocks, int steps, bool masked) {
    constexpr double WG_COST = 6.0, SPLIT_COST = 55.0;
    constexpr int XCDS = 8, MAX_SPLITS_PER_BLOCK = 16, MIN_RANGE = 32;
    const int n_cu = cu_count();
    BwdCut cut;
    cut.blocks_per_xcd = (blocks + XCDS - 1) / XCDS;
    cut.splits2 = 1;
    // unequal work-groups only even out when there are enough of them; a small masked launch
    // is priced like a dense one (which is also right when its mask hides nothing)
    const bool ragged = masked && blocks >= 2 * n_cu;
    const double work = ragged ? 0.5 * steps : (double)steps;
    auto cost = [&](int S) {
        const double rounds = ragged ? (double)blocks * S / n_cu
                                     : (double)(((int64_t)blocks * S + n_cu - 1) / n_cu);
        return rounds * (work / S + WG_COST) + (S > 1 ? SPLIT_COST : 0.0);
    };
    int best = 1;
    double best_cost = cost(1);
    for (int S = 2; S <= 8; ++S) {
        if (steps / S < MIN_RANGE) break;
        const double c = cost(S);
        if (c < best_cost) { best_cost = c; best = S; }
    }
    cut.splits = best;
    cut.whole = best == 1 ? cut.blocks_per_xcd : 0;
    cut.mid = cut.blocks_per_xcd - cut.whole;
    // Equal blocks, more of them than CUs: whole rounds of unsplit blocks first (no partial sums,
    // one ramp per block), and only the blocks past the last whole round are cut - all alike into
    // as many ranges as fill their rounds best, or in two groups that make one round each: as
    // many blocks as give every CU one work-group when cut in S1 = ceil(CUs / blocks), and what
    // is left then in as many ranges as the CUs can take.
    const int cu_x = n_cu / XCDS;
    if (!ragged && cu_x > 0 && cut.blocks_per_xcd > cu_x && blocks % XCDS == 0) {
        const int full = cut.blocks_per_xcd / cu_x * cu_x, rest = cut.blocks_per_xcd - full;
        if (rest == 0) return cut;       // (best is 1 then)
        const double whole_cost = (full / cu_x) * (steps + WG_COST) + SPLIT_COST;
        for (int S = 2; S <= 8; ++S) {
            if (steps / S < MIN_RANGE) break;
            const double c = whole_cost + ((rest * S + cu_x - 1) / cu_x) * ((double)steps / S + WG_COST);
            if (c < best_cost) { best_cost = c; cut.whole = full; cut.mid = rest; cut.splits = S; cut.splits2 = 1; }
        }
        const int S1 = (cu_x + rest - 1) / rest;
        const int n1 = std::min(rest, cu_x / S1), left = rest - n1;
        if (S1 >= 2 && steps / S1 >= MIN_RANGE && left > 0) {
            int S2 = std::min(std::min(cu_x / left, MAX_SPLITS_PER_BLOCK), steps / MIN_RANGE);
            if (S2 >= 2) {
                const double c = whole_cost + ((double)steps / S1 + WG_COST) + ((double)steps / S2 + WG_COST);
                if (c < best_cost) { best_cost = c; cut.whole = full; cut.mid = n1; cut.splits = S1; cut.splits2 = S2; }
            }
        }
    }
    return cut;
}

static size_t dkv_scratch_bytes(const lvx_attn_shape* s) {
    return (size_t)2 * s->B * s->Lkv * s->Hkv * s->D * sizeof(float);
}

// The dQ GEMM of a small row window (a one-round launch, or few rows against many tokens) has
// fewer C tiles than the chip has compute units; its
// contraction over the tokens is then split over several work-groups that store fp32
// partial tiles, each split into its own slice of a scratch; the slices are summed and
// rounded to bf16 afterwards (fp32 atomics into one slice were measured slower).  Returns
// the number of splits (1: none) and the tokens per split.
static int dq_k_splits(const lvx_attn_shape* s, int32_t row_count, int* split_len) {
    const int tile_rows = s->kv_start ? 256 : 512;      // as launch_gemm picks them
    const int tiles = row_count > 256 ? (row_count + tile_rows - 1) / tile_rows : 1;
    const int wgs = s->B * s->Hq * tiles;
    const int blocks = (s->Lkv + 127) / 128;
    int ks = 1;
    const int n_cu = cu_count();
    if (wgs <= n_cu / 2) ks = std::min(std::min(8, n_cu / wgs), blocks);
    const int per = (blocks + ks - 1) / ks;
    *split_len = per * 128;
    return (blocks + per - 1) / per;
}

// Regions of the backward workspace, in order: dS^T tiles; fp32 dK/dV scratch (split-steps mode
// with bf16 outputs); row metadata records (2 floats per row and head); fp32 dQ partial tiles,
// one slice per split (split dQ contraction only); with an interval mask the live-tile tables (group hulls, runs
// of live tiles per token block, the groups ranked by hull length).  Every region is a multiple of 16 bytes.
struct BwdWorkspace {
    size_t ds, dkv, meta, dq32, hull, runs, order, total;
    int n_tiles, group, n_groups;
};

static BwdWorkspace bwd_workspace(const lvx_attn_shape* s, int32_t row_count) {
    BwdWorkspace w{};
    const size_t tokens = ((size_t)s->Lkv + 127) / 128 * 128;
    const size_t rows = ((size_t)row_count + 31) / 32 * 32;
    auto up16 = [](size_t n) { return (n + 15) / 16 * 16; };
    w.n_tiles = (int)(rows / 32);
    w.group = 8;                            // row tiles per M tile of the masked dQ GEMM (256 rows)
    w.n_groups = (w.n_tiles + w.group - 1) / w.group;
    size_t off = 0;
    w.ds = off; off += (size_t)s->B * s->Hq * tokens * rows * sizeof(uint16_t);
    w.dkv = off; off += dkv_scratch_bytes(s);
    w.meta = off; off += (size_t)s->B * s->Hq * rows * 2 * sizeof(float);
    int sl;
    w.dq32 = off;
    const int ks = dq_k_splits(s, row_count, &sl);
    if (ks > 1) off += (size_t)ks * s->B * s->Hq * rows * s->D * sizeof(float);
    if (s->kv_start) {
        const size_t nkb = tokens / 128;
        w.hull = off; off += up16((size_t)s->B * w.n_groups * 2 * sizeof(int32_t));
        w.runs = off; off += (size_t)s->B * nkb * 8 * sizeof(int32_t);
        w.order = off; off += up16((size_t)s->B * w.n_groups * sizeof(int32_t));
    }
    w.total = off;
    return w;
}

size_t lvx_bwd_workspace_bytes(const lvx_attn_shape* s, int32_t row_count) {
    if (!s || row_count <= 0) return 0;
    return bwd_workspace(s, row_count).total;
}

int lvx_bwd(const lvx_attn_shape* s, const lvx_tensor* q, const lvx_tensor* k, const lvx_tensor* v,
            const lvx_tensor* dout, const float* lse, const float* delta, const lvx_tensor* dq,
            const lvx_tensor* dk, const lvx_tensor* dv, int32_t dkv_accumulate,
            int32_t row_begin, int32_t row_count, void* workspace, size_t workspace_bytes, void* stream) {
    LVX_TRY(check_shape(s));
    LVX_TRY(check_tensor(q));
    LVX_TRY(check_tensor(k));
    LVX_TRY(check_tensor(v));
    LVX_TRY(check_tensor(dout));
    LVX_TRY(check_tensor(dq));
    LVX_TRY(check_tensor(dk));
    LVX_TRY(check_tensor(dv));
    if (!lse || !delta) return LVX_ERR_NULL;
    if (dkv_accumulate != 0 && dkv_accumulate != 1) return LVX_ERR_SHAPE;
    LVX_TRY(check_rows(s, row_begin, row_count));
    if (row_count == 0) return LVX_OK;
    // row offsets inside a tensor are formed in 32 bits
    if ((int64_t)s->Lq * q->stride_s >= (int64_t)1 << 31 || (int64_t)s->Lq * dout->stride_s >= (int64_t)1 << 31)
        return LVX_ERR_UNSUPPORTED;
    if (!workspace || workspace_bytes < lvx_bwd_workspace_bytes(s, row_count)) return LVX_ERR_WORKSPACE;
    if (!aligned16(workspace)) return LVX_ERR_ALIGN;
    hipStream_t st = static_cast<hipStream_t>(stream);

    BwdParams p{};
    p.f16 = s->dtype == LVX_F16;
    p.D = s->D;
    p.q = static_cast<const uint16_t*>(q->ptr);
    p.k = static_cast<const uint16_t*>(k->ptr);
    p.v = static_cast<const uint16_t*>(v->ptr);
    p.dout = static_cast<const uint16_t*>(dout->ptr);
    p.dk = dk->ptr; p.dv = dv->ptr;
    p.qs = st3(q); p.ks = st3(k); p.vs = st3(v); p.dos = st3(dout); p.dks = st3(dk); p.dvs = st3(dv);
    p.kv_len = s->kv_len; p.kv_start = s->kv_start; p.kv_end = s->kv_end;
    p.bias = s->bias; p.bias_b = s->bias_stride_b; p.bias_h = s->bias_stride_h; p.bias_r = s->bias_stride_r;
    p.B = s->B; p.Hq = s->Hq; p.Hkv = s->Hkv; p.Lq = s->Lq; p.Lkv = s->Lkv; p.G = s->Hq / s->Hkv;
    p.row_begin = row_begin; p.row_end = row_begin + row_count;
    p.n_kv_blocks = (s->Lkv + 127) / 128;
    p.scale = s->scale; p.scale_log2e = s->scale * LOG2E;
    const int64_t tokens = (int64_t)p.n_kv_blocks * 128;
    const int64_t rows = ((int64_t)row_count + 31) / 32 * 32;
    p.ds_ws = static_cast<uint16_t*>(workspace);
    p.ws_ld = rows * 128;          // one token block: (rows / 32) tiles of 128 x 32
    p.ws_bh = tokens * rows;

    const BwdWorkspace wsl = bwd_workspace(s, row_count);
    char* const wsb = static_cast<char*>(workspace);
    // how the launch is shaped decides which fp32 scratches it accumulates into; the
    // metadata kernel zeroes them on its way
    const int blocks = s->B * s->Hkv * p.n_kv_blocks;
    const int steps = p.G * (int)(rows / 32);
    const BwdCut cut = choose_bwd_cut(blocks, steps, s->kv_start != nullptr);
    p.n_blocks = blocks;
    p.blocks_per_xcd = cut.blocks_per_xcd;
    p.whole_blocks = cut.whole;
    p.mid_blocks = cut.mid;
    p.q_splits = cut.splits;
    p.q_splits2 = cut.splits2;
    p.dkv_mode = cut.any_split() ? 2 : (dkv_accumulate ? 1 : 0);
    float* const scratch = (cut.any_split() && !dkv_accumulate) ? reinterpret_cast<float*>(wsb + wsl.dkv) : nullptr;
    int split_len = 0;
    const int ks = dq_k_splits(s, row_count, &split_len);
    float* const dq32 = ks > 1 ? reinterpret_cast<float*>(wsb + wsl.dq32) : nullptr;
    {
        float* meta = reinterpret_cast<float*>(wsb + wsl.meta);
        MetaParams mp{lse, delta, meta, s->B, s->Hq, s->Lq, row_begin, row_begin + row_count, (int)(rows / 32), s->scale};
        mp.zero_dst[0] = reinterpret_cast<uint32_t*>(scratch);
        mp.zero_n16[0] = scratch ? (int64_t)(dkv_scratch_bytes(s) / 16) : 0;
        hipError_t em = launch_bwd_meta(mp, st);
        if (em != hipSuccess) return static_cast<int>(em);
        p.meta = meta;
    }
    int32_t* hull = nullptr;
    int32_t* order = nullptr;
    if (s->kv_start) {
        // interval mask: token blocks skip the row tiles that see none of their tokens
        hull = reinterpret_cast<int32_t*>(wsb + wsl.hull);
        // the ranking is quadratic in the number of groups; where there are that many, the dQ
        // GEMM's work-groups even out in index order
        if (ks <= 1 && s->B * wsl.n_groups <= MAX_RANKED_GROUPS) order = reinterpret_cast<int32_t*>(wsb + wsl.order);
        LiveParams lp{s->kv_len, s->kv_start, s->kv_end, hull, reinterpret_cast<int32_t*>(wsb + wsl.runs), order,
                      s->B, s->Lq, s->Lkv, row_begin,
                      row_begin + row_count, wsl.n_tiles, wsl.group, wsl.n_groups, p.n_kv_blocks};
        hipError_t el = launch_bwd_live(lp, st);
        if (el != hipSuccess) return static_cast<int>(el);
        p.live_runs = lp.live_runs;
    }

    const int64_t dkv_elems = (int64_t)s->B * s->Lkv * s->Hkv * s->D;
    // blocks with one work-group are written by it as the caller asked
    p.dk_whole = p.dk; p.dv_whole = p.dv;
    p.dks_whole = p.dks; p.dvs_whole = p.dvs;
    p.whole_mode = dkv_accumulate ? 1 : 0;
    if (scratch) {
        // bf16 outputs, several work-groups per token block: those blocks are summed in the fp32
        // scratch [2][B, Lkv, Hkv, D] and rounded once afterwards
        p.dk = scratch;
        p.dv = scratch + dkv_elems;
        p.dks = p.dvs = Strides3{(int64_t)s->Lkv * s->Hkv * s->D, (int64_t)s->D, (int64_t)s->Hkv * s->D};
    }
    hipError_t e = launch_bwd(p, s->kv_start != nullptr, st);
    if (e != hipSuccess) return static_cast<int>(e);
    if (scratch) {
        // scratch memory order is [B, Lkv, Hkv, D]: cast with (H, L) = (Lkv, Hkv); dK and dV in one launch
        CastParams cp{};
        cp.f16 = p.f16;
        cp.D = s->D;
        cp.src = scratch;
        cp.dst = static_cast<uint16_t*>(dk->ptr);
        cp.ds = Strides3{dk->stride_b, dk->stride_s, dk->stride_h};
        cp.src2 = scratch + dkv_elems;
        cp.dst2 = static_cast<uint16_t*>(dv->ptr);
        cp.ds2 = Strides3{dv->stride_b, dv->stride_s, dv->stride_h};
        cp.B = s->B; cp.H = s->Lkv; cp.L = s->Hkv;
        if (p.whole_blocks > 0) {
            cp.skip_bpx = p.blocks_per_xcd; cp.skip_whole = p.whole_blocks;
            cp.skip_nkvb = p.n_kv_blocks; cp.skip_nblocks = p.n_blocks;
        }
        e = launch_cast(cp, st);
        if (e != hipSuccess) return static_cast<int>(e);
    }

    // dQ[b, h, rows, :] = dS^T[b, h]^T (rows x tokens) * K[b, h / G] (tokens x D), scale already in dS
    GemmParams g{};
    g.f16 = p.f16;
    GemmProblem& pr = g.prob[0];
    pr.A[0] = p.ds_ws; pr.lda[0] = rows;
    pr.Bm[0] = p.k; pr.ldb[0] = k->stride_s;
    pr.K[0] = s->Lkv; pr.nseg = 1;
    pr.C = static_cast<uint16_t*>(dq->ptr) + (int64_t)row_begin * dq->stride_s;
    pr.ldc = dq->stride_s;
    g.M_ld = (int)rows;
    g.batch_inner = s->Hq;
    g.b_group = p.G;
    g.a_batch = p.ws_bh;
    g.b_outer = k->stride_b; g.b_inner = k->stride_h;
    g.c_outer = dq->stride_b; g.c_inner = dq->stride_h;
    g.k_len = s->kv_len;
    g.a_tiled_m = (int)(rows / 32);
    g.k_range = hull;            // [B][M tiles][2]: the group hulls are per M tile of this GEMM
    g.m_order = order;
    fill_grid(g, row_count, s->D, 1, s->B * s->Hq);
    if (ks <= 1) return static_cast<int>(launch_gemm(g, true, true, st));
    // split contraction: every split stores its partial tiles in its own fp32 slice; the
    // cast sums the slices and rounds into dq
    g.k_splits = ks; g.k_split_len = split_len;
    g.c32 = dq32; g.c32_batch = (int64_t)row_count * s->D; g.c32_ld = row_count;   // [split][B * Hq][D][row_count]
    g.c32_split = (int64_t)s->B * s->Hq * g.c32_batch;
    e = launch_gemm(g, true, true, st);
    if (e != hipSuccess) return static_cast<int>(e);
    CastParams cq{};
    cq.f16 = p.f16;
    cq.D = s->D;
    cq.src = dq32;
    cq.dst = static_cast<uint16_t*>(dq->ptr) + (int64_t)row_begin * dq->stride_s;
    cq.ds = st3(dq);
    cq.B = s->B; cq.H = s->Hq; cq.L = row_count;
    cq.transposed = 1;
    cq.nsum = ks; cq.sum_stride = g.c32_split;
    return static_cast<int>(launch_cast(cq, st));
}

static int check_dtype(int32_t dtype) { return (dtype == LVX_BF16 || dtype == LVX_F16) ? LVX_OK : LVX_ERR_DTYPE; }

int lvx_cast_f32(const float* src, const lvx_tensor* dst, int32_t B, int32_t H, int32_t L, int32_t D,
                 int32_t dtype, void* stream) {
    LVX_TRY(check_dtype(dtype));
    if (!src) return LVX_ERR_NULL;
    LVX_TRY(check_tensor(dst));
    if (!aligned16(src)) return LVX_ERR_ALIGN;
    if (D != 128 && D != 64 && D != 32 && D != 16) return LVX_ERR_HEAD_DIM;
    if (B <= 0 || H <= 0 || L <= 0) return LVX_ERR_SHAPE;
    CastParams p{};
    p.f16 = dtype == LVX_F16;
    p.D = D;
    p.src = src;
    p.dst = static_cast<uint16_t*>(dst->ptr);
    p.ds = st3(dst);
    p.B = B; p.H = H; p.L = L;
    return static_cast<int>(launch_cast(p, static_cast<hipStream_t>(stream)));
}

static int check_gemm_ptr(const void* p, int64_t ld) {
    if (!p) return LVX_ERR_NULL;
    if (!aligned16(p) || (ld % 8) != 0) return LVX_ERR_ALIGN;
    if (ld <= 0 || ld >= (1 << 21)) return LVX_ERR_SHAPE;   // 32-bit byte offsets inside a tile
    return LVX_OK;
}

}  // extern "C"

static void fill_grid(GemmParams& g, int M, int N, int nprob, int nbatch = 1) {
    g.M = M; g.N = N; g.nprob = nprob;
    if (g.M_ld < M) g.M_ld = M;
    g.nbatch = nbatch;
    if (g.batch_inner < 1) g.batch_inner = 1;
    if (g.b_group < 1) g.b_group = 1;
}

extern "C" {

static int kv_proj_impl(const void* x, int64_t ldx, const void* w_k, const void* w_v, int64_t ldw, int32_t w_in_major,
                        void* k_out, void* v_out, int64_t ldkv, int32_t M, int32_t Dm, int32_t N,
                        const void* k_norm_w, float eps, void* k_raw, float* k_rstd, int32_t dtype, void* stream) {
    LVX_TRY(check_dtype(dtype));
    LVX_TRY(check_gemm_ptr(x, ldx));
    LVX_TRY(check_gemm_ptr(w_k, ldw));
    LVX_TRY(check_gemm_ptr(k_out, ldkv));
    if (!w_v != !v_out) return LVX_ERR_NULL;       // both or neither
    const int np = w_v ? 2 : 1;                    // one projection only: the Q side
    if (np == 2) {
        LVX_TRY(check_gemm_ptr(w_v, ldw));
        LVX_TRY(check_gemm_ptr(v_out, ldkv));
    }
    if (M <= 0 || Dm <= 0 || N <= 0 || (Dm % 8) || (N % 8)) return LVX_ERR_SHAPE;
    if (ldx < Dm || ldkv < N || ldw < (w_in_major ? N : Dm)) return LVX_ERR_SHAPE;
    GemmParams g{};
    g.f16 = dtype == LVX_F16;
    const void* w[2] = {w_k, w_v};
    void* c[2] = {k_out, v_out};
    for (int i = 0; i < np; ++i) {
        GemmProblem& pr = g.prob[i];
        pr.A[0] = static_cast<const uint16_t*>(x); pr.lda[0] = ldx;
        pr.Bm[0] = static_cast<const uint16_t*>(w[i]); pr.ldb[0] = ldw;
        pr.K[0] = Dm; pr.nseg = 1;
        pr.C = static_cast<uint16_t*>(c[i]); pr.ldc = ldkv;
    }
    if (k_norm_w) {
        if (N % 128) return LVX_ERR_HEAD_DIM;      // the norm runs over heads of 128 columns
        if (!aligned16(k_norm_w)) return LVX_ERR_ALIGN;
        if (!(eps >= 0.f)) return LVX_ERR_SHAPE;
        if (k_raw) LVX_TRY(check_gemm_ptr(k_raw, ldkv));
        if (k_rstd && (reinterpret_cast<uintptr_t>(k_rstd) & 3)) return LVX_ERR_ALIGN;
        g.norm_w = static_cast<const uint16_t*>(k_norm_w);
        g.norm_eps = eps;
        g.c_raw = static_cast<uint16_t*>(k_raw);
        g.rstd = k_rstd;
    }
    fill_grid(g, M, N, np);
    return static_cast<int>(launch_gemm(g, false, w_in_major != 0, static_cast<hipStream_t>(stream)));
}

int lvx_kv_proj(const void* x, int64_t ldx, const void* w_k, const void* w_v, int64_t ldw, int32_t w_in_major,
                void* k_out, void* v_out, int64_t ldkv, int32_t M, int32_t Dm, int32_t N, int32_t dtype, void* stream) {
    return kv_proj_impl(x, ldx, w_k, w_v, ldw, w_in_major, k_out, v_out, ldkv, M, Dm, N, nullptr, 0.f, nullptr,
                        nullptr, dtype, stream);
}

int lvx_kv_proj_norm(const void* x, int64_t ldx, const void* w_k, const void* w_v, int64_t ldw, int32_t w_in_major,
                     void* k_out, void* v_out, int64_t ldkv, int32_t M, int32_t Dm, int32_t N,
                     const void* k_norm_w, float eps, void* k_raw, float* k_rstd, int32_t dtype, void* stream) {
    if (!k_norm_w) return LVX_ERR_NULL;
    return kv_proj_impl(x, ldx, w_k, w_v, ldw, w_in_major, k_out, v_out, ldkv, M, Dm, N, k_norm_w, eps, k_raw,
                        k_rstd, dtype, stream);
}

int lvx_k_norm_bwd(const void* dk, int64_t lddk, const void* k_raw, int64_t ldk, const float* k_rstd,
                   const void* k_norm_w, void* dk_raw, int64_t lddk_raw, float* dw, int32_t M, int32_t N,
                   int32_t dtype, void* stream) {
    LVX_TRY(check_dtype(dtype));
    LVX_TRY(check_gemm_ptr(dk, lddk));
    LVX_TRY(check_gemm_ptr(k_raw, ldk));
    LVX_TRY(check_gemm_ptr(dk_raw, lddk_raw));
    if (!k_rstd || !k_norm_w) return LVX_ERR_NULL;
    if (!aligned16(k_norm_w) || (reinterpret_cast<uintptr_t>(k_rstd) & 3) || (reinterpret_cast<uintptr_t>(dw) & 3))
        return LVX_ERR_ALIGN;
    if (M <= 0 || N <= 0) return LVX_ERR_SHAPE;
    if (N % 128) return LVX_ERR_HEAD_DIM;
    if (lddk < N || ldk < N || lddk_raw < N) return LVX_ERR_SHAPE;
    NormBwdParams p{};
    p.f16 = dtype == LVX_F16;
    p.dy = static_cast<const uint16_t*>(dk);
    p.x = static_cast<const uint16_t*>(k_raw);
    p.rstd = k_rstd;
    p.w = static_cast<const uint16_t*>(k_norm_w);
    p.dx = static_cast<uint16_t*>(dk_raw);
    p.dw = dw;
    p.ldy = lddk; p.ldx = ldk; p.lddx = lddk_raw;
    p.M = M; p.heads = N / 128;
    return static_cast<int>(launch_norm_bwd(p, static_cast<hipStream_t>(stream)));
}

int lvx_dx_vis(const void* dk, const void* dv, int64_t lddkv, const void* w_k, const void* w_v, int64_t ldw,
               int32_t w_in_major, void* dx, int64_t lddx, int32_t M, int32_t Dm, int32_t N, int32_t dtype,
               void* stream) {
    LVX_TRY(check_dtype(dtype));
    LVX_TRY(check_gemm_ptr(dk, lddkv));
    LVX_TRY(check_gemm_ptr(w_k, ldw));
    LVX_TRY(check_gemm_ptr(dx, lddx));
    if (!dv != !w_v) return LVX_ERR_NULL;          // both or neither
    if (dv) {
        LVX_TRY(check_gemm_ptr(dv, lddkv));
        LVX_TRY(check_gemm_ptr(w_v, ldw));
    }
    if (M <= 0 || Dm <= 0 || N <= 0 || (Dm % 8) || (N % 8)) return LVX_ERR_SHAPE;
    if (lddkv < N || lddx < Dm || ldw < (w_in_major ? N : Dm)) return LVX_ERR_SHAPE;
    GemmParams g{};
    g.f16 = dtype == LVX_F16;
    GemmProblem& pr = g.prob[0];
    pr.A[0] = static_cast<const uint16_t*>(dk); pr.A[1] = static_cast<const uint16_t*>(dv);
    pr.lda[0] = pr.lda[1] = lddkv;
    pr.Bm[0] = static_cast<const uint16_t*>(w_k); pr.Bm[1] = static_cast<const uint16_t*>(w_v);
    pr.ldb[0] = pr.ldb[1] = ldw;
    pr.K[0] = N; pr.K[1] = dv ? N : 0; pr.nseg = dv ? 2 : 1;
    pr.C = static_cast<uint16_t*>(dx); pr.ldc = lddx;
    fill_grid(g, M, Dm, 1);
    // B[k = n][col = dm]: W [Dm][N] has k contiguous, W [N][Dm] has the column contiguous
    return static_cast<int>(launch_gemm(g, false, w_in_major == 0, static_cast<hipStream_t>(stream)));
}

int lvx_dw_kv(const void* x, int64_t ldx, const void* dk, const void* dv, int64_t lddkv, void* dw_k, void* dw_v,
              int64_t ldw, int32_t w_in_major, int32_t M, int32_t Dm, int32_t N, int32_t dtype, void* stream) {
    LVX_TRY(check_dtype(dtype));
    LVX_TRY(check_gemm_ptr(x, ldx));
    LVX_TRY(check_gemm_ptr(dk, lddkv));
    LVX_TRY(check_gemm_ptr(dw_k, ldw));
    if (!dv != !dw_v) return LVX_ERR_NULL;         // both or neither
    const int np = dv ? 2 : 1;
    if (np == 2) {
        LVX_TRY(check_gemm_ptr(dv, lddkv));
        LVX_TRY(check_gemm_ptr(dw_v, ldw));
    }
    if (M <= 0 || Dm <= 0 || N <= 0 || (Dm % 8) || (N % 8)) return LVX_ERR_SHAPE;
    if (ldx < Dm || lddkv < N || ldw < (w_in_major ? N : Dm)) return LVX_ERR_SHAPE;
    GemmParams g{};
    g.f16 = dtype == LVX_F16;
    const void* d[2] = {dk, dv};
    void* c[2] = {dw_k, dw_v};
    for (int i = 0; i < np; ++i) {
        GemmProblem& pr = g.prob[i];
        if (w_in_major) {   // dW [Dm][N] = X^T dK
            pr.A[0] = static_cast<const uint16_t*>(x); pr.lda[0] = ldx;
            pr.Bm[0] = static_cast<const uint16_t*>(d[i]); pr.ldb[0] = lddkv;
        } else {            // dW [N][Dm] = dK^T X
            pr.A[0] = static_cast<const uint16_t*>(d[i]); pr.lda[0] = lddkv;
            pr.Bm[0] = static_cast<const uint16_t*>(x); pr.ldb[0] = ldx;
        }
        pr.K[0] = M; pr.nseg = 1;
        pr.C = static_cast<uint16_t*>(c[i]); pr.ldc = ldw;
    }
    if (w_in_major) fill_grid(g, Dm, N, np);
    else fill_grid(g, N, Dm, np);
    return static_cast<int>(launch_gemm(g, true, true, static_cast<hipStream_t>(stream)));
}

}  // extern "C"
