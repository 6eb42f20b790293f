// Shared host/device helpers of libfgnn_hip.so (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include "fgnn.h"

#define FGNN_WPB 4      // waves per workgroup: every wave works on its own item
#define FGNN_TPB 256

// ------------------------------------------------------------------ host side
void fgnn_set_error(const char *fmt, ...);

#define FGNN_REQUIRE(cond, code, ...)            \
    do {                                         \
        if (!(cond)) {                           \
            fgnn_set_error(__VA_ARGS__);         \
            return (code);                       \
        }                                        \
    } while (0)

#define FGNN_HIP(call)                                                        \
    do {                                                                      \
        hipError_t err__ = (call);                                            \
        if (err__ != hipSuccess) {                                            \
            fgnn_set_error("%s failed: %s", #call, hipGetErrorString(err__)); \
            return (int)err__;                                                \
        }                                                                     \
    } while (0)

static inline int fgnn_launch_status(const char *what)
{
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        fgnn_set_error("launch of %s failed: %s", what, hipGetErrorString(err));
        return (int)err;
    }
    return 0;
}

static inline bool fgnn_aligned16(const void *p) { return (((uintptr_t)p) & 15u) == 0; }
static inline size_t fgnn_align256(size_t x) { return (x + 255) & ~(size_t)255; }
// Fills n floats with v on `st` (a kernel, so it may be captured into a HIP graph).
int fgnn_fill_f32(float *p, size_t n, float v, hipStream_t st);
int fgnn_current_device_has_xcd_mapping();      // 1: workgroup w of a dispatch runs on XCD w % FGNN_NUM_XCD on the current device

// Stable LSD radix sort of (key, payload) pairs and an inclusive int32 scan (fgnn_csr2csc.hip); device pointers.
size_t fgnn_rs_sort_workspace(int64_t n);
int fgnn_rs_key_bits(int n_keys);
int fgnn_rs_sort_pairs(const int *keys_in, const int *pay_in, int64_t n, int key_bits, int *pay_out, const int **sorted_keys, void *workspace,
                       hipStream_t st);
size_t fgnn_scan_workspace(int64_t n);
int fgnn_inclusive_scan_i32(const int *in, int64_t n, int *out, int *tile_sums, int *total_dev, hipStream_t st);

// One work item: the edge range [begin, end) of `row`.  slot < 0: the item covers the whole
// row and writes final results; slot >= 0: a segment of a split row, written as partial `slot`.
struct fgnn_item { int row, begin, end, slot; };
// A split row: its partials are slots [first_slot, first_slot + nseg).
struct fgnn_split { int row, first_slot, nseg, pad; };

struct fgnn_schedule {
    int n_rows;
    int64_t n_edges;
    int seg_len;
    int n_items;
    int n_partials;
    int n_split;
    fgnn_item *items_dev;
    fgnn_split *split_dev;
    const int32_t *ptr_dev;
    int device;
    // XCD-aware schedules only: the index array with every row's entries grouped by source bucket
    // (a per-row permutation of the caller's index array), else NULL
    int n_buckets;
    const int32_t *idx_src_dev;
    int32_t *bidx_dev;
    int32_t *bpos_dev;      // original position of every bucket-ordered entry (for per-edge arrays)
    int own_order;          // the position map was handed to the caller: per-edge arrays come in the schedule's entry order
    // Every item at a slot >= n_wave_slots has at most FGNN_GROUP_ITEM_MAX entries (the lists are sorted longest first, so the
    // long items are a prefix).  A multiple of 64 slots per source bucket, or n_items.  Kernels that give each lane group of a
    // wave its own item start there; the prefix goes to the kernels that put a whole wave on an item.
    int n_wave_slots;
};
#define FGNN_GROUP_ITEM_MAX 64
// The index array a kernel walks under schedule `s`, and the map from its positions back to the
// caller's edge positions (NULL = identity).
static inline const int32_t *fgnn_sched_idx(const fgnn_schedule *s, const int32_t *idx) { return (s && s->n_buckets > 0) ? s->bidx_dev : idx; }
static inline const int32_t *fgnn_sched_pos(const fgnn_schedule *s) { return (s && s->n_buckets > 0) ? s->bpos_dev : nullptr; }
// false for an XCD-aware schedule built without the position map: operators with per-edge tensors must refuse it
static inline bool fgnn_sched_has_pos(const fgnn_schedule *s) { return !s || s->n_buckets == 0 || s->n_edges == 0 || s->bpos_dev != nullptr || s->own_order; }

#define FGNN_NUM_XCD 8      // workgroup w of a dispatch runs on XCD w % 8 (gfx942 / gfx950, SPX mode)
// Source bucket of a node id: the top 3 bits of a multiplicative hash, so hot ids spread evenly.
static __host__ __device__ inline int fgnn_bucket_of(int id) { return (int)(((uint32_t)id * 2654435761u) >> 29); }

// Feature-row layout of the gather kernels: a row of `HF` floats is spread over the 64 lanes
// of a wave in R slabs of 64*VEC floats; VEC = 4 uses 128-bit loads.
struct fgnn_rowcfg { int vec; int r; bool full; };
static inline bool fgnn_pick_rowcfg(int HF, int F, bool aligned, fgnn_rowcfg *c)
{
    int vec = (aligned && (F % 4 == 0)) ? 4 : 1;
    int per = 64 * vec;
    int need = (HF + per - 1) / per;
    int r = 1;
    while (r < need) r *= 2;
    if ((vec == 4 && r > 4) || (vec == 1 && r > 16)) return false;
    c->vec = vec; c->r = r; c->full = (HF == per * r);
    return true;
}


// Calls f.template operator()<VEC, R, FULL>() for the row layout chosen at run time.
template <typename Fn>
static inline int fgnn_dispatch_rowcfg(const fgnn_rowcfg &c, Fn &&f)
{
    if (c.vec == 4) {
        if (c.r == 1) return c.full ? f.template operator()<4, 1, true>() : f.template operator()<4, 1, false>();
        if (c.r == 2) return c.full ? f.template operator()<4, 2, true>() : f.template operator()<4, 2, false>();
        return c.full ? f.template operator()<4, 4, true>() : f.template operator()<4, 4, false>();
    }
    switch (c.r) {
    case 1: return f.template operator()<1, 1, false>();
    case 2: return f.template operator()<1, 2, false>();
    case 4: return f.template operator()<1, 4, false>();
    case 8: return f.template operator()<1, 8, false>();
    default: return f.template operator()<1, 16, false>();
    }
}

// ------------------------------------------------------------------ device side
#ifdef __HIPCC__
__device__ __forceinline__ int fg_lane() { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }
__device__ __forceinline__ int fg_wave() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }
__device__ __forceinline__ int fg_uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ float fg_readlane(float v, int l) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l)); }
__device__ __forceinline__ float fg_bperm(float v, int src_lane) { return __int_as_float(__builtin_amdgcn_ds_bpermute(src_lane << 2, __float_as_int(v))); }

// Marks a wave-uniform address as such for the compiler: the halves go through readfirstlane (free
// for values that already sit in scalar registers), which keeps the address arithmetic before it on
// the scalar unit and lets `base + 32-bit lane offset` loads use the scalar-base addressing mode.
typedef float fg_f4 __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(1))) char *fg_gptr;        // a pointer known to be to global memory
__device__ __forceinline__ fg_gptr fg_uniform_ptr(const void *p)
{
    uint64_t a = (uint64_t)p;
    uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a), hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32));
    return (fg_gptr)(((uint64_t)hi << 32) | lo);
}
// The empty asm re-defines a 32-bit lane offset inside the block it is called from.  Loads of that block
// then show instruction selection "scalar base + zero-extended 32-bit offset" and get the scalar-base
// form, with no address arithmetic on the vector unit (a zero-extension hoisted out of the loop hides it).
__device__ __forceinline__ uint32_t fg_pin(uint32_t off) { asm volatile("" : "+v"(off)); return off; }

template <int CTRL>
__device__ __forceinline__ float fg_dpp(float v)
{
    // every control used here is a permutation inside a row, so no lane lacks a source; "old = 0,
    // bound_ctrl" lets the compiler fold the move into the add / max that consumes it
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
// Butterfly inside each row of 16 lanes (quad xor 1, quad xor 2, half-row mirror, row mirror),
// then the four row results are combined through scalar registers.  All lanes get the result.
__device__ __forceinline__ float fg_wave_max(float v)
{
    v = fmaxf(v, fg_dpp<0xB1>(v));
    v = fmaxf(v, fg_dpp<0x4E>(v));
    v = fmaxf(v, fg_dpp<0x141>(v));
    v = fmaxf(v, fg_dpp<0x140>(v));
    float a = fg_readlane(v, 0), b = fg_readlane(v, 16), c = fg_readlane(v, 32), d = fg_readlane(v, 48);
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}
__device__ __forceinline__ float fg_wave_sum(float v)
{
    v = v + fg_dpp<0xB1>(v);
    v = v + fg_dpp<0x4E>(v);
    v = v + fg_dpp<0x141>(v);
    v = v + fg_dpp<0x140>(v);
    float a = fg_readlane(v, 0), b = fg_readlane(v, 16), c = fg_readlane(v, 32), d = fg_readlane(v, 48);
    return (a + b) + (c + d);
}
// Orders LDS traffic between the lanes of ONE wave (each wave owns a private LDS region, LDS
// instructions of a wave execute in order, so only the compiler has to be held back).
__device__ __forceinline__ void fg_wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__device__ __forceinline__ float fg_lrelu(float x, float slope) { return x > 0.f ? x : x * slope; }
// max(x, 0) of a finite x as one integer maximum on the bit pattern (negative floats are negative integers)
__device__ __forceinline__ float fg_relu_bits(float x) { return __int_as_float(max(__float_as_int(x), 0)); }
// SLE1: the slope is known to lie in [0, 1], where LeakyReLU(x) == max(x, slope*x)
template <bool SLE1>
__device__ __forceinline__ float fg_lrelu_t(float x, float slope) { return SLE1 ? fmaxf(x, x * slope) : (x > 0.f ? x : x * slope); }
#define FGNN_LOG2E 1.4426950408889634f
#define FGNN_LN2 0.6931471805599453f

template <int VEC> struct fg_vec;
template <> struct fg_vec<4> {
    float4 v;
    __device__ __forceinline__ void zero() { v = make_float4(0.f, 0.f, 0.f, 0.f); }
    __device__ __forceinline__ void load(const float *p) { v = *reinterpret_cast<const float4 *>(p); }
    // wave-uniform base + unsigned 32-bit byte offset: lets the load use a scalar base register
    __device__ __forceinline__ void load_off(const char *base, uint32_t off) { v = *reinterpret_cast<const float4 *>(base + off); }
    __device__ __forceinline__ void load_off(fg_gptr base, uint32_t off) { fg_f4 t = *(const __attribute__((address_space(1))) fg_f4 *)(base + off); v = make_float4(t.x, t.y, t.z, t.w); }
    __device__ __forceinline__ void store(float *p) const { *reinterpret_cast<float4 *>(p) = v; }
    // streaming store: the line is not kept in L2 (results nobody gathers again in this kernel)
    __device__ __forceinline__ void store_nt(float *p) const { __builtin_nontemporal_store(v.x, p); __builtin_nontemporal_store(v.y, p + 1); __builtin_nontemporal_store(v.z, p + 2); __builtin_nontemporal_store(v.w, p + 3); }
    __device__ __forceinline__ void fma(float w, const fg_vec &x) { v.x = fmaf(w, x.v.x, v.x); v.y = fmaf(w, x.v.y, v.y); v.z = fmaf(w, x.v.z, v.z); v.w = fmaf(w, x.v.w, v.w); }
    __device__ __forceinline__ void add(const fg_vec &x) { v.x += x.v.x; v.y += x.v.y; v.z += x.v.z; v.w += x.v.w; }
    __device__ __forceinline__ void scale(float w) { v.x *= w; v.y *= w; v.z *= w; v.w *= w; }
    // a*this + b*o
    __device__ __forceinline__ fg_vec lin(float a, float b, const fg_vec &o) const { fg_vec r; r.v.x = a * v.x + b * o.v.x; r.v.y = a * v.y + b * o.v.y; r.v.z = a * v.z + b * o.v.z; r.v.w = a * v.w + b * o.v.w; return r; }
    __device__ __forceinline__ float dot(const fg_vec &o) const { return (v.x * o.v.x + v.y * o.v.y) + (v.z * o.v.z + v.w * o.v.w); }
};
template <> struct fg_vec<1> {
    float v;
    __device__ __forceinline__ void zero() { v = 0.f; }
    __device__ __forceinline__ void load(const float *p) { v = *p; }
    __device__ __forceinline__ void load_off(const char *base, uint32_t off) { v = *reinterpret_cast<const float *>(base + off); }
    __device__ __forceinline__ void load_off(fg_gptr base, uint32_t off) { v = *(const __attribute__((address_space(1))) float *)(base + off); }
    __device__ __forceinline__ void store(float *p) const { *p = v; }
    __device__ __forceinline__ void store_nt(float *p) const { __builtin_nontemporal_store(v, p); }
    __device__ __forceinline__ void fma(float w, const fg_vec &x) { v = fmaf(w, x.v, v); }
    __device__ __forceinline__ void add(const fg_vec &x) { v += x.v; }
    __device__ __forceinline__ void scale(float w) { v *= w; }
    __device__ __forceinline__ fg_vec lin(float a, float b, const fg_vec &o) const { fg_vec r; r.v = a * v + b * o.v; return r; }
    __device__ __forceinline__ float dot(const fg_vec &o) const { return v * o.v; }
};

// Which floats of a feature row a lane owns: slab r covers floats [eoff[r], eoff[r]+VEC) which
// all belong to head hd[r]; ok[r] is false past the end of the row.
template <int VEC, int R>
struct fg_lanemap {
    int eoff[R];
    int hd[R];
    bool ok[R];
    __device__ __forceinline__ void init(int lane, int HF, int F)
    {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            eoff[r] = (lane + 64 * r) * VEC;
            ok[r] = eoff[r] < HF;
            hd[r] = ok[r] ? eoff[r] / F : 0;
        }
    }
    // Head-aligned variant for kernels that reduce inside heads with DPP: head h takes lanes
    // [h*lphp, (h+1)*lphp) (lphp a power of two >= F/VEC), the lanes past F/VEC of a head stay idle.
    __device__ __forceinline__ void init_padded(int lane, int H, int F, int lphp)
    {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int li = lane + 64 * r;
            int h = li / lphp, sub = li - h * lphp;
            ok[r] = h < H && sub * VEC < F;
            hd[r] = ok[r] ? h : 0;
            eoff[r] = ok[r] ? h * F + sub * VEC : 0;
        }
    }
};

// Decode the work item of this wave.  Returns false when there is none.
__device__ __forceinline__ bool fg_get_item(const fgnn_item *items, int n_items, const int *ptr,
                                            int &row, int &b, int &e, int &slot)
{
    int item = fg_uni((int)blockIdx.x * FGNN_WPB + fg_wave());
    if (item >= n_items) return false;
    if (items) {
        fgnn_item it = items[item];
        row = fg_uni(it.row); b = fg_uni(it.begin); e = fg_uni(it.end); slot = fg_uni(it.slot);
        if (row < 0) return false;         // padding item of an XCD-aware schedule
    } else {
        row = item; b = fg_uni(ptr[item]); e = fg_uni(ptr[item + 1]); slot = -1;
    }
    return true;
}

// The slot of a work list that lane group g of the wave takes when every group has an item of its own: the G slots of a
// wave are consecutive among the slots of ONE source bucket (slot ((k / WPB) * 8 + b) * WPB + k % WPB is the k-th slot of
// bucket b in an XCD-aware list, and workgroup w runs on XCD w % 8); in a plain list they are simply consecutive.
// `first`: the slot the lane-group part of the launch starts at (fgnn_schedule::n_wave_slots); `w`: the workgroup's index
// in that part (the workgroups before it take the head of the list a wave per item; their number is a multiple of 8 when the
// list is XCD-aware, so w % 8 is still the workgroup's XCD).
__device__ __forceinline__ int fg_group_slot(int G, int g, int bucketed, int first, int w)
{
    const int v = fg_wave();
    if (!bucketed) return first + (w * FGNN_WPB + v) * G + g;
    const int b = w % FGNN_NUM_XCD, k = first / FGNN_NUM_XCD + ((w / FGNN_NUM_XCD) * FGNN_WPB + v) * G + g;
    return ((k / FGNN_WPB) * FGNN_NUM_XCD + b) * FGNN_WPB + k % FGNN_WPB;
}

// Grid of the kernels that give every lane group of a wave its own work item (fg_group_slot): one wave per `pack` slots of
// the list, the slots of a wave from one source bucket when the list is XCD-aware (its length is then a multiple of
// 8 * FGNN_WPB).
static inline unsigned fgnn_group_item_grid(int n_items, int pack, bool bucketed)
{
    const int64_t waves = ((int64_t)n_items + pack - 1) / pack;
    unsigned grid = (unsigned)((waves + FGNN_WPB - 1) / FGNN_WPB);
    if (bucketed) grid = (grid + FGNN_NUM_XCD - 1) / FGNN_NUM_XCD * FGNN_NUM_XCD;
    return grid;
}

// Weighted accumulation of up to 64 gathered feature rows with the weights staged in LDS (the
// stored-weight SpMM and the GMMConv forward; the fused GAT kernels stream instead).  Lane t of
// `idv` holds the node id of edge t of the chunk (lanes >= cnt hold any valid id), wl[h*64 + t] its
// weight for head h (0 for lanes >= cnt).  Node ids are moved to scalar registers so that every row
// is fetched by one base-plus-lane-offset 128-bit load per slab, 8 rows in flight.
template <int VEC, int R, bool FULL>
__device__ __forceinline__ void fg_accum_chunk(const float *__restrict__ feat, int HF, int idv, int cnt,
                                               const float *wl, const fg_lanemap<VEC, R> &lm, fg_vec<VEC> (&T)[R])
{
    constexpr int U = (R >= 8) ? 1 : 8 / R;
    for (int t = 0; t < cnt; t += U) {
        fg_vec<VEC> ld[U][R];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            int id = __builtin_amdgcn_readlane(idv, t + u);
            const float *base = feat + (size_t)id * (size_t)HF;
#pragma unroll
            for (int r = 0; r < R; ++r) ld[u][r].load(base + ((FULL || lm.ok[r]) ? lm.eoff[r] : 0));   // idle lanes re-read float 0: no branch
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float w[U];
            if constexpr (U % 4 == 0) {
#pragma unroll
                for (int u = 0; u < U; u += 4) {
                    float4 q = *reinterpret_cast<const float4 *>(wl + lm.hd[r] * 64 + t + u);
                    w[u] = q.x; w[u + 1] = q.y; w[u + 2] = q.z; w[u + 3] = q.w;
                }
            } else if constexpr (U == 2) {
                float2 q = *reinterpret_cast<const float2 *>(wl + lm.hd[r] * 64 + t);
                w[0] = q.x; w[1] = q.y;
            } else {
                w[0] = wl[lm.hd[r] * 64 + t];
            }
#pragma unroll
            for (int u = 0; u < U; ++u) T[r].fma(w[u], ld[u][r]);
        }
    }
}

// Sum over groups of LPH consecutive lanes (LPH a power of two <= 64, groups aligned); every lane
// of a group gets the group's sum.  Steps inside a row of 16 lanes are DPP, wider ones go through
// the LDS crossbar.
template <int LPH>
__device__ __forceinline__ float fg_group_sum(float v)
{
    if constexpr (LPH >= 2) v += fg_dpp<0xB1>(v);
    if constexpr (LPH >= 4) v += fg_dpp<0x4E>(v);
    if constexpr (LPH >= 8) v += fg_dpp<0x141>(v);
    if constexpr (LPH >= 16) v += fg_dpp<0x140>(v);
    if constexpr (LPH >= 32) v += fg_bperm(v, fg_lane() ^ 16);
    if constexpr (LPH >= 64) v += fg_bperm(v, fg_lane() ^ 32);
    return v;
}
// Lanes per head for which the kernels have a DPP reduction; 0 selects the generic LDS path.
static inline int fgnn_pick_lph(int vec, int F)
{
    int lph = F / vec;
    if (vec == 4 && (lph == 1 || lph == 2 || lph == 4 || lph == 8 || lph == 16 || lph == 32)) return lph;
    return 0;
}
// Lanes per head of the head-aligned lane map (fg_lanemap::init_padded) for a width that is a multiple
// of 4 but whose quarter is not a power of two; 0 when the dense map already is head-aligned or the
// padded row would not fit 4 slabs.
static inline int fgnn_pad_lph(int vec, int H, int F)
{
    if (vec != 4 || F % 4 != 0) return 0;
    int l = 1;
    while (l * 4 < F) l *= 2;
    if (l * 4 == F || l > 32 || (int64_t)H * l * 4 > 1024) return 0;
    return l;
}
// Entries of a narrow row gathered per load instruction (1 = one row per wave).
static inline int fgnn_pick_pack(int vec, int HF)
{
    if (vec != 4) return 1;
    return HF <= 32 ? 8 : HF <= 64 ? 4 : HF <= 128 ? 2 : 1;
}
// Calls f.template operator()<LPH>() for a value returned by fgnn_pick_lph.
template <typename Fn>
static inline int fgnn_dispatch_lph(int lph, Fn &&f)
{
    switch (lph) {
    case 1: return f.template operator()<1>();
    case 2: return f.template operator()<2>();
    case 4: return f.template operator()<4>();
    case 8: return f.template operator()<8>();
    case 16: return f.template operator()<16>();
    case 32: return f.template operator()<32>();
    default: return f.template operator()<0>();
    }
}

// Per-head sums of per-lane partial values: lane h (< H) returns the sum over the F/VEC
// lane-slabs of head h.  `scr` is wave-private LDS of at least 64*R floats.
template <int VEC, int R>
__device__ __forceinline__ float fg_head_reduce(float *scr, const float (&part)[R], const fg_lanemap<VEC, R> &lm,
                                                int lane, int H, int F)
{
#pragma unroll
    for (int r = 0; r < R; ++r)
        if (lm.ok[r]) scr[lane + 64 * r] = part[r];
    fg_wave_lds_sync();
    float acc = 0.f;
    if (lane < H) {
        int n = F / VEC;
        for (int k = 0; k < n; ++k) acc += scr[lane * n + k];
    }
    fg_wave_lds_sync();
    return acc;
}
// The same sums for a handful of heads without LDS: one masked wave sum per head.
#define FGNN_FEW_HEADS 8
template <int VEC, int R>
__device__ __forceinline__ float fg_head_reduce_few(const float (&part)[R], const fg_lanemap<VEC, R> &lm, int lane, int H)
{
    float res = 0.f;
    for (int h = 0; h < H; ++h) {
        float v = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) v += (lm.ok[r] && lm.hd[r] == h) ? part[r] : 0.f;
        float s = fg_wave_sum(v);
        if (lane == h) res = s;
    }
    return res;
}
// Rows narrower than a wave (H*F <= 128 floats): G = 2, 4 or 8 entries of the row are gathered by
// one load instruction.  The wave is cut into G groups of LPR = 64/G lanes; group g takes entries
// g, g+G, ... of a chunk, lane `sub` of a group owns floats [4*sub, 4*sub+4) of the feature row.  Each
// group keeps its own partial sums; a butterfly over the groups adds them up at the end.
template <int G>
struct fg_packmap {
    static constexpr int LPR = 64 / G;
    int grp, eoff, hd;
    bool ok;
    __device__ __forceinline__ void init(int lane, int HF, int F)
    {
        grp = lane / LPR;
        eoff = (lane % LPR) * 4;
        ok = eoff < HF;
        hd = ok ? eoff / F : 0;
    }
    __device__ __forceinline__ void init_padded(int lane, int H, int F, int lphp)      // see fg_lanemap::init_padded
    {
        grp = lane / LPR;
        int li = lane % LPR;
        int h = li / lphp, sub = li - h * lphp;
        ok = h < H && sub * 4 < F;
        hd = ok ? h : 0;
        eoff = ok ? h * F + sub * 4 : 0;
    }
};
// Sum over the G groups; every group ends with the total.
template <int G>
__device__ __forceinline__ void fg_pack_reduce(fg_vec<4> &T, int lane)
{
#pragma unroll
    for (int step = 64 / G; step < 64; step <<= 1) {
        T.v.x += fg_bperm(T.v.x, lane ^ step); T.v.y += fg_bperm(T.v.y, lane ^ step);
        T.v.z += fg_bperm(T.v.z, lane ^ step); T.v.w += fg_bperm(T.v.w, lane ^ step);
    }
}
#endif  // __HIPCC__
