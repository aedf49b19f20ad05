// Optimizer-step kernels for gfx950 (MI355X) behind the C ABI of include/elx_abi.h.
//
// All passes are streaming, HBM-bound element-wise work; there is no contraction, so no MFMA.
//
//   grad_stats_kernel   one read of the low-precision gradients -> overflow flag + sum of squares
//                       per chunk (fp32 per-lane partials over 32-128 elements, flushed into an
//                       fp64 accumulator; wave shuffle -> LDS -> one partial per workgroup;
//                       a second tiny launch folds the partials in a fixed order)
//   adam_step_kernel    unscale + Adam/AdamW on master/m/v + low-precision writeback, tile by tile
//   refresh_kernel      the low-precision refresh alone (padding runs, skipped steps, state loading,
//                       the gather source copy of a host-resident shard)
//   land_grads_kernel   payload or per-tensor gradients -> shard (copy / cast), with the overflow
//                       flag and sum of squares of what lands riding the copy; stats_fold_kernel and
//                       stats_finish_kernel fold its per-workgroup partials
//
// Shape of the update launch, as measured on MI355X.  The update moves 14 B in and 14 B out per
// element over four in-place regions.  HBM serves such a read/write mix best when the set of
// addresses in flight is a tight, orderly moving window that is only just deep enough to cover
// the memory latency; deeper queues cost bandwidth (full occupancy: ~5.5 TB/s; about 40 KB in
// flight per compute unit: 6.7 TB/s; a plain copy peaks at ~6.65 TB/s the same way, write-only
// traffic falls from 7.2 to 6.2 TB/s between a shallow and a full queue).  Hence:
//   * one wavefront per workgroup, one 256-element tile per workgroup (one access per stream per
//     lane), tiles handed out in address order by the dispatcher (a persistent grid-stride loop is
//     much slower here, and so are wider workgroups or more accesses per lane);
//   * the common case is one straight line of code: with two or three wavefronts per SIMD there
//     is nothing to hide a branch, a conditional load or a late table lookup behind;
//   * every access is a fully coalesced 128-bit (fp32) / 64-bit (16-bit types) per-lane access,
//     so one wavefront instruction covers one contiguous 1 KiB / 512 B span;
//   * the number of resident workgroups per compute unit is capped through a dynamic LDS
//     reservation (default 13 for 16-bit gradients, 12 for fp32 ones), not by the register file;
//   * loads carry the non-temporal hint, stores go out non-temporal at agent scope.
//
// Arithmetic contract (what the parity tests pin): fp32 throughout, IEEE division and square
// root, the only fused multiply-adds are the three written as fmaf(); compile with
// -ffp-contract=off.  The op order is torch.optim.Adam's single-tensor path
// (torch/optim/adam.py:414-419, 457, 476, 528-545) with the fused forms its CPU kernels use.
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <atomic>

#include "elx_abi.h"
#include "elx_host.h"

using namespace elx_host;

// Partials workspace of elx_grad_stats_mt_static, the one entry point that takes no workspace from
// its caller and allocates none: every GPU the library runs on holds this array until the process
// ends.  In host code the name is only a handle for hipGetSymbolAddress; launches get the address
// that call returned for the current device (scratch_of_current_device below).  No kernel names the
// array: the compiler keeps it, and gives it the external linkage the runtime's lookup needs, because
// host code names it (an explicit `used` attribute would keep it internal and the lookup would fail).
constexpr uint32_t kStaticPartials = 65536;    // ElxStats records: 1 MiB
static __device__ __align__(256) unsigned char scratch[kStaticPartials * sizeof(ElxStats)];

namespace {

constexpr uint32_t kStatsStreamBlocksPerCu = 3;        // stats workgroups (256 threads) per CU when the set streams from HBM

constexpr int kStatsThreads = 256;
constexpr int kStatsUnroll = 4;
constexpr uint32_t kMaxStatsBlocks = 1024;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------------------------------------
// element codecs
// ---------------------------------------------------------------------------------------------

template <int D>
struct Elem;

template <>
struct Elem<ELX_F32> {
    typedef float scalar;
    typedef f32x4 vec4;
    static __device__ __forceinline__ float to_f32(float x) { return x; }
    static __device__ __forceinline__ float from_f32(float x) { return x; }
};

template <>
struct Elem<ELX_F16> {
    typedef uint16_t scalar;
    typedef u16x4 vec4;
    static __device__ __forceinline__ float to_f32(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
    // v_cvt_f16_f32: round to nearest even, overflow to inf, subnormals kept
    static __device__ __forceinline__ uint16_t from_f32(float x) {
        return __builtin_bit_cast(uint16_t, (_Float16)x);
    }
};

template <>
struct Elem<ELX_BF16> {
    typedef uint16_t scalar;
    typedef u16x4 vec4;
    static __device__ __forceinline__ float to_f32(uint16_t b) {
        return __builtin_bit_cast(float, (uint32_t)b << 16);
    }
    // v_cvt_pk_bf16_f32: round to nearest even, NaN stays a quiet NaN
    static __device__ __forceinline__ uint16_t from_f32(float x) { return __builtin_bit_cast(uint16_t, (__bf16)x); }
};

// KEEP: an ordinary load, which leaves the line in the memory-side cache for a launch that reads it
// again soon; otherwise non-temporal (read once, do not displace anything).
template <bool KEEP, typename V>
__device__ __forceinline__ V ld_stream(const V *p) {
    if constexpr (KEEP)
        return *p;
    else
        return __builtin_nontemporal_load(p);
}

// Tile-local buffer addressing for the update launch: each stream of a tile is described by a
// raw buffer resource (uniform base = start of the tile, extent = the tile), and a lane addresses
// it with a 32-bit byte offset.  Loads carry the non-temporal hint; stores go out non-temporal at
// agent scope.  Being compiler intrinsics (not inline assembly) they keep the compiler's own
// hazard and wait-count handling.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
constexpr int kAuxLoad = 2;          // nt
constexpr int kAuxStore = 2 | 16;    // nt | sc1
constexpr int kAuxStoreKeep = 16;    // sc1

__device__ __forceinline__ __amdgpu_buffer_rsrc_t tile_rsrc(const void *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

template <typename V>
struct TileIo;

template <>
struct TileIo<f32x4> {
    template <int AUX = kAuxLoad>
    static __device__ __forceinline__ f32x4 load(__amdgpu_buffer_rsrc_t r, uint32_t off) {
        return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, AUX));
    }
    template <int AUX = kAuxStore>
    static __device__ __forceinline__ void store(__amdgpu_buffer_rsrc_t r, uint32_t off, f32x4 x) {
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, x), r, (int)off, 0, AUX);
    }
};

template <>
struct TileIo<u16x4> {
    template <int AUX = kAuxLoad>
    static __device__ __forceinline__ u16x4 load(__amdgpu_buffer_rsrc_t r, uint32_t off) {
        return __builtin_bit_cast(u16x4, __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, AUX));
    }
    template <int AUX = kAuxStore>
    static __device__ __forceinline__ void store(__amdgpu_buffer_rsrc_t r, uint32_t off, u16x4 x) {
        __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, x), r, (int)off, 0, AUX);
    }
};

// Cache policy of an update launch (ELX_FLAG_KEEP_CACHED, ELX_FLAG_KEEP_STATE_CACHED).
//   kStream     every access streams: non-temporal loads, non-temporal stores at agent scope;
//   kKeepLowp   the low-precision copy alone is stored at agent scope without the non-temporal hint: such a
//               store is taken in by the memory-side cache, over the gradient it replaces when that is still
//               there, and written back from there later;
//   kKeepState  everything the launch touches fits that cache: ordinary loads, and all stores as above, so
//               that the next step finds the state there.
enum { kStream = 0, kKeepLowp = 1, kKeepState = 2 };
template <int POLICY>
struct Aux {
    static constexpr int load = POLICY == kKeepState ? 0 : kAuxLoad;
    static constexpr int store = POLICY == kKeepState ? kAuxStoreKeep : kAuxStore;
    static constexpr int store_lowp = POLICY == kStream ? kAuxStore : kAuxStoreKeep;
};

// ---------------------------------------------------------------------------------------------
// the update of one element
// ---------------------------------------------------------------------------------------------

struct Hyper {
    float decay_mul, l2_wd, lerp_w, beta2, omb2, bc2_sqrt, eps, neg_step;
    uint32_t flags;
    float gate_div, gate_inv;    // only loaded by the gated launch
    uint32_t gate;               // mode | skip << 8
};

template <bool GATED = false>
__device__ __forceinline__ Hyper load_hyper(const ElxHyper *__restrict__ h) {
    Hyper r;
    if constexpr (GATED) {
        r.gate_div = h->gate_div_scale;
        r.gate_inv = h->gate_inv_scale;
        r.gate = h->gate;
    } else {
        r.gate_div = -1.0f;
        r.gate_inv = 1.0f;
        r.gate = 0;
    }
    r.decay_mul = h->decay_mul;
    r.l2_wd = h->l2_wd;
    r.lerp_w = h->lerp_w;
    r.beta2 = h->beta2;
    r.omb2 = h->omb2;
    r.bc2_sqrt = h->bc2_sqrt;
    r.eps = h->eps;
    r.neg_step = h->neg_step;
    r.flags = h->flags;
    return r;
}

// (how the gradient is unscaled -- kDivNone / kDivMulInv / kDivTrue and struct Unscale -- is declared in elx_host.h)

// One element, with the three launch-uniform choices (unscale mode, L2 vs decoupled decay, which
// end the lerp starts from) fixed at compile time: the tile loop below is then straight-line code.
// With only two or three wavefronts per SIMD there is nothing to hide a branch behind.
template <int MODE, bool L2, bool LERP_FROM_G>
__device__ __forceinline__ void adam_elem_fixed(float g, float &p, float &m, float &v, const Hyper &h,
                                                const Unscale &us) {
    if (MODE == kDivMulInv)
        g = g * us.inv_scale;
    else if (MODE == kDivTrue)
        g = g / us.div_scale;
    p = p * h.decay_mul;                                   // AdamW: p *= 1 - lr*wd (1.0f otherwise)
    if (L2) g = fmaf(h.l2_wd, p, g);                       // L2: g += wd*p
    const float diff = g - m;
    m = fmaf(h.lerp_w, diff, LERP_FROM_G ? g : m);         // m.lerp_(g, 1-beta1)
    v = fmaf(h.omb2 * g, g, v * h.beta2);                  // v.mul_(beta2).addcmul_(g, g, 1-beta2)
    const float denom = sqrtf(v) / h.bc2_sqrt + h.eps;     // sqrt(v)/sqrt(bc2) + eps
    p = p + (h.neg_step * m) / denom;                      // p.addcdiv_(m, denom, -lr/bc1)
}

// The same element with the choices read at run time (the element-by-element path).
__device__ __forceinline__ void adam_elem(float g, float &p, float &m, float &v, const Hyper &h, const Unscale &us) {
    if (us.mode == kDivMulInv)
        g = g * us.inv_scale;
    else if (us.mode == kDivTrue)
        g = g / us.div_scale;
    p = p * h.decay_mul;
    if (h.flags & ELX_HYPER_L2) g = fmaf(h.l2_wd, p, g);
    const float diff = g - m;
    const float base = (h.flags & ELX_HYPER_LERP_FROM_G) ? g : m;
    m = fmaf(h.lerp_w, diff, base);
    v = fmaf(h.omb2 * g, g, v * h.beta2);
    const float denom = sqrtf(v) / h.bc2_sqrt + h.eps;
    p = p + (h.neg_step * m) / denom;
}

template <int GD, int MODE, bool L2, bool LERP_FROM_G>
__device__ __forceinline__ void tile_math(const typename Elem<GD>::vec4 (&G)[kUnroll], f32x4 (&P)[kUnroll],
                                          f32x4 (&M)[kUnroll], f32x4 (&V)[kUnroll], const Hyper &h, const Unscale &us) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
        for (int k = 0; k < kVec; ++k) {
            float g = Elem<GD>::to_f32(G[u][k]);
            float p = P[u][k], m = M[u][k], v = V[u][k];
            adam_elem_fixed<MODE, L2, LERP_FROM_G>(g, p, m, v, h, us);
            P[u][k] = p;
            M[u][k] = m;
            V[u][k] = v;
        }
    }
}

template <int GD, int MODE>
__device__ __forceinline__ void tile_math_flags(const typename Elem<GD>::vec4 (&G)[kUnroll], f32x4 (&P)[kUnroll],
                                                f32x4 (&M)[kUnroll], f32x4 (&V)[kUnroll], const Hyper &h,
                                                const Unscale &us) {
    const bool l2 = h.flags & ELX_HYPER_L2, from_g = h.flags & ELX_HYPER_LERP_FROM_G;
    if (!l2 && !from_g)
        tile_math<GD, MODE, false, false>(G, P, M, V, h, us);
    else if (l2 && !from_g)
        tile_math<GD, MODE, true, false>(G, P, M, V, h, us);
    else if (!l2 && from_g)
        tile_math<GD, MODE, false, true>(G, P, M, V, h, us);
    else
        tile_math<GD, MODE, true, true>(G, P, M, V, h, us);
}

// ---------------------------------------------------------------------------------------------
// fused update + writeback
// ---------------------------------------------------------------------------------------------

template <int LD, int POLICY>
__device__ __forceinline__ void store_lowp_vec(const ElxChunk &c, uint64_t base, const f32x4 (&P)[kUnroll]) {
    if constexpr (LD != ELX_NONE) {
        if (!c.lowp_out) return;
        typedef typename Elem<LD>::vec4 lvec;
        typedef typename Elem<LD>::scalar lscalar;
        const __amdgpu_buffer_rsrc_t lr = tile_rsrc(reinterpret_cast<lscalar *>(c.lowp_out) + base, kTile * sizeof(lscalar));
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            lvec L;
#pragma unroll
            for (int k = 0; k < kVec; ++k) L[k] = Elem<LD>::from_f32(P[u][k]);
            TileIo<lvec>::template store<Aux<POLICY>::store_lowp>(lr, (threadIdx.x + u * kWave) * sizeof(lvec), L);
        }
    }
}

// Whole tile outside the valid head of the shard (padding), or the writeback-only launch.
template <int LD, int POLICY>
__device__ __forceinline__ void tile_refresh_vec(const ElxChunk &c, uint64_t base) {
    if constexpr (LD != ELX_NONE) {
        if (!c.lowp_out) return;
        const __amdgpu_buffer_rsrc_t pr = tile_rsrc(c.master + base, kTile * sizeof(float));
        f32x4 P[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
            P[u] = TileIo<f32x4>::template load<Aux<POLICY>::load>(pr, (threadIdx.x + u * kWave) * sizeof(f32x4));
        store_lowp_vec<LD, POLICY>(c, base, P);
    }
}

// Any tile: element by element, each element looking up the segment that covers it.  Used for
// tiles that straddle a segment boundary, the partial tile at the end of a chunk, and buffers
// whose base pointers are not 16-byte aligned.  `s` is the first segment whose end is > base.
template <int GD, int LD, bool GATED>
__device__ __forceinline__ void tile_scalar(const ElxChunk &c, uint64_t base, uint32_t tile_n, uint32_t s,
                                            const ElxSeg *__restrict__ segs, const ElxHyper *__restrict__ hypers,
                                            const Unscale &us_arg, bool refresh_only) {
    typedef typename Elem<GD>::scalar gscalar;
    const gscalar *grad = reinterpret_cast<const gscalar *>(c.grad);
    for (uint32_t i = threadIdx.x; i < tile_n; i += kWave) {
        const uint64_t e = base + i;
        float p = c.master[e];
        if (!refresh_only) {
            uint32_t cs = s;
            while (cs < c.seg_end && segs[cs].end <= e) ++cs;
            if (cs < c.seg_end && segs[cs].begin <= e) {
                const Hyper h = load_hyper<GATED>(hypers + segs[cs].hyper);
                Unscale us = us_arg;
                bool skip = false;
                if constexpr (GATED) {
                    us.div_scale = h.gate_div;
                    us.inv_scale = h.gate_inv;
                    us.mode = (int)(h.gate & 0xFFu);
                    skip = (h.gate >> 8) != 0;
                }
                if (!skip) {
                    float g = grad ? Elem<GD>::to_f32(grad[e]) : 0.0f;
                    float m = c.m[e], v = c.v[e];
                    adam_elem(g, p, m, v, h, us);
                    c.master[e] = p;
                    c.m[e] = m;
                    c.v[e] = v;
                }
            }
        }
        if constexpr (LD != ELX_NONE) {
            if (c.lowp_out) reinterpret_cast<typename Elem<LD>::scalar *>(c.lowp_out)[e] = Elem<LD>::from_f32(p);
        }
    }
}

// Fetches a whole chunk record with one round trip of scalar loads.  Left to itself the compiler
// loads the fields in the order the branches below first need them, which costs three dependent
// trips to the scalar cache before the first vector load of the tile can be issued.
__device__ __forceinline__ ElxChunk load_chunk_row(const ElxChunk *__restrict__ row) {
    const uint64_t *w = reinterpret_cast<const uint64_t *>(row);
    uint64_t w0 = w[0], w1 = w[1], w2 = w[2], w3 = w[3], w4 = w[4], w5 = w[5], w6 = w[6], w7 = w[7], w8 = w[8];
    asm volatile("" : "+s"(w0), "+s"(w1), "+s"(w2), "+s"(w3), "+s"(w4), "+s"(w5), "+s"(w6), "+s"(w7), "+s"(w8));
    ElxChunk c;
    c.grad = reinterpret_cast<const void *>(w0);
    c.lowp_out = reinterpret_cast<void *>(w1);
    c.master = reinterpret_cast<float *>(w2);
    c.m = reinterpret_cast<float *>(w3);
    c.v = reinterpret_cast<float *>(w4);
    c.n_alloc = w5;
    c.n_valid = w6;
    c.tile_begin = w7;
    c.seg_begin = (uint32_t)w8;
    c.seg_end = (uint32_t)(w8 >> 32);
    return c;
}
static_assert(sizeof(ElxChunk) == 72, "load_chunk_row reads nine 64-bit words");

// The update and landing launches pass a dynamic LDS size that no kernel ever touches: it only caps how
// many workgroups share a compute unit (occupancy_reservation below).

// GATED: the unscale parameters and the skip flag are read from the hyper records (where elx_decide
// has put them earlier on the same stream) instead of the kernel arguments, so that the launch can be
// enqueued before the host knows whether the step happens.  They arrive with the hyper record the
// tile loads anyway; on a skip the tile only refreshes its low-precision copy.
template <int GD, int LD, bool GATED, int POLICY>
__device__ __forceinline__ void adam_step_tile(const ElxChunk *__restrict__ chunks, const ElxSeg *__restrict__ segs,
                                               const ElxHyper *__restrict__ hypers, Unscale us, uint32_t scalar_only) {
    // 2-D grid (tiles, records): blockIdx.y names the record, blockIdx.x the tile; nothing is looked
    // up, and workgroups beyond a record's last tile exit
    const uint32_t ci = blockIdx.y, local_tile = blockIdx.x;
    const ElxChunk c = load_chunk_row(chunks + ci);
    const uint64_t base = (uint64_t)local_tile * kTile;
    if (base >= c.n_alloc) return;    // a shorter record

    typedef typename Elem<GD>::vec4 gvec;
    typedef typename Elem<GD>::scalar gscalar;

    // ---- the common case: a whole tile inside the valid head of the shard ---------------------
    // Kept as one straight line (loads, table lookups, arithmetic, stores): with two or three
    // wavefronts per SIMD there is nothing to hide a detour behind.
    if (!scalar_only && base + kTile <= c.n_valid) {
        const __amdgpu_buffer_rsrc_t pr = tile_rsrc(c.master + base, kTile * sizeof(float));
        const __amdgpu_buffer_rsrc_t mr = tile_rsrc(c.m + base, kTile * sizeof(float));
        const __amdgpu_buffer_rsrc_t vr = tile_rsrc(c.v + base, kTile * sizeof(float));
        // a NULL gradient reads as zero: an empty buffer returns 0 for every lane, without a branch
        const __amdgpu_buffer_rsrc_t gr =
            c.grad ? tile_rsrc(reinterpret_cast<const gscalar *>(c.grad) + base, kTile * sizeof(gscalar))
                   : tile_rsrc(c.master, 0);
        gvec G[kUnroll];
        f32x4 P[kUnroll], M[kUnroll], V[kUnroll];
        // issue every load of the tile before looking at the segment table: the table lookups
        // below then overlap the memory latency
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            G[u] = TileIo<gvec>::template load<Aux<POLICY>::load>(gr, (threadIdx.x + u * kWave) * sizeof(gvec));
            const uint32_t off = (threadIdx.x + u * kWave) * sizeof(f32x4);
            P[u] = TileIo<f32x4>::template load<Aux<POLICY>::load>(pr, off);
            M[u] = TileIo<f32x4>::template load<Aux<POLICY>::load>(mr, off);
            V[u] = TileIo<f32x4>::template load<Aux<POLICY>::load>(vr, off);
        }
        // first segment of the chunk that ends after the start of the tile
        uint32_t s = c.seg_begin, s_hi = c.seg_end;
        while (s < s_hi) {
            const uint32_t mid = (s + s_hi) >> 1;
            if (segs[mid].end > base)
                s_hi = mid;
            else
                s = mid + 1;
        }
        const bool has = s < c.seg_end;
        const uint64_t sb = has ? segs[s].begin : ~0ull;
        const uint64_t se = has ? segs[s].end : 0ull;
        if (has && sb <= base && se >= base + kTile) {
            const Hyper h = load_hyper<GATED>(hypers + segs[s].hyper);
            if constexpr (GATED) {
                us.div_scale = h.gate_div;
                us.inv_scale = h.gate_inv;
                us.mode = (int)(h.gate & 0xFFu);
                if (h.gate >> 8) {    // the step is skipped: refresh the low-precision copy only
                    store_lowp_vec<LD, POLICY>(c, base, P);
                    return;
                }
            }
            if (us.mode == kDivMulInv)
                tile_math_flags<GD, kDivMulInv>(G, P, M, V, h, us);
            else if (us.mode == kDivTrue)
                tile_math_flags<GD, kDivTrue>(G, P, M, V, h, us);
            else
                tile_math_flags<GD, kDivNone>(G, P, M, V, h, us);
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const uint32_t off = (threadIdx.x + u * kWave) * sizeof(f32x4);
                TileIo<f32x4>::template store<Aux<POLICY>::store>(pr, off, P[u]);
                TileIo<f32x4>::template store<Aux<POLICY>::store>(mr, off, M[u]);
                TileIo<f32x4>::template store<Aux<POLICY>::store>(vr, off, V[u]);
            }
            store_lowp_vec<LD, POLICY>(c, base, P);
            return;
        }
        if (!has || sb >= base + kTile) {    // inside the valid head but owned by no segment
            store_lowp_vec<LD, POLICY>(c, base, P);
            return;
        }
        // the tile straddles a segment boundary: redo it element by element below
    }

    // ---- everything else ------------------------------------------------------------------------
    const uint64_t left = c.n_alloc - base;
    const uint32_t tile_n = left < kTile ? (uint32_t)left : kTile;
    if (base >= c.n_valid) {    // padding inside an update chunk: refresh only
        if (tile_n == kTile && !scalar_only)
            tile_refresh_vec<LD, POLICY>(c, base);
        else
            tile_scalar<GD, LD, GATED>(c, base, tile_n, 0, segs, hypers, us, true);
        return;
    }
    uint32_t s = c.seg_begin, s_hi = c.seg_end;
    while (s < s_hi) {
        const uint32_t mid = (s + s_hi) >> 1;
        if (segs[mid].end > base)
            s_hi = mid;
        else
            s = mid + 1;
    }
    tile_scalar<GD, LD, GATED>(c, base, tile_n, s, segs, hypers, us, false);
}

template <int GD, int LD, bool GATED, int POLICY>
__global__ __launch_bounds__(kWave) void adam_step_kernel(const ElxChunk *__restrict__ chunks,
                                                          const ElxSeg *__restrict__ segs,
                                                          const ElxHyper *__restrict__ hypers, Unscale us,
                                                          uint32_t scalar_only) {
    adam_step_tile<GD, LD, GATED, POLICY>(chunks, segs, hypers, us, scalar_only);
}

// A handful of hyper records travel in the arguments of the launch that uses them.
constexpr uint32_t kMaxArgHypers = 32;
struct HyperPack {
    ElxHyper h[kMaxArgHypers];
};
static_assert(offsetof(HyperPack, h) == 0, "the records start at offset 0 of the argument segment");

// The update launch of a host-decided or standalone step whose hyper records fit its own arguments:
// the table the tiles read is the argument segment itself, so no launch has to fill a table first.
template <int GD, int LD, int POLICY>
__global__ __launch_bounds__(kWave) void adam_step_args_kernel(HyperPack pack, const ElxChunk *__restrict__ chunks,
                                                               const ElxSeg *__restrict__ segs, Unscale us,
                                                               uint32_t scalar_only) {
    // `pack` is the first argument: the records are read where they lie (indexing the by-value
    // aggregate would copy it to private memory first)
    typedef const ElxHyper __attribute__((address_space(4))) *kernarg_hypers;
    const ElxHyper *hypers = (const ElxHyper *)(kernarg_hypers)__builtin_amdgcn_kernarg_segment_ptr();
    adam_step_tile<GD, LD, false, POLICY>(chunks, segs, hypers, us, scalar_only);
}

// ---------------------------------------------------------------------------------------------
// low-precision refresh alone
// ---------------------------------------------------------------------------------------------

// lowp_out[0, n_alloc) = round-to-nearest-even(master) for every chunk.  4 bytes in, 2 bytes out per
// element.  The same shape as the landing launch (which, for an fp32 payload and a 16-bit shard, is
// this copy plus the flags): one wavefront per workgroup, one piece of four 128-bit loads per lane,
// residency capped through the LDS reservation, pieces handed out in address order.  Grid
// (blocks_per_chunk, n_chunks); a workgroup takes several pieces only when a record has more pieces
// than the grid has blocks.
constexpr int kRefreshThreads = kWave;
constexpr int kRefreshUnroll = 4;
constexpr uint32_t kRefreshPiece = kRefreshThreads * kVec * kRefreshUnroll;    // 1024 elements
constexpr uint32_t kRefreshBlocksPerCu = 13;
constexpr uint32_t kMaxRefreshBlocks = 1u << 20;

template <int LD>
__device__ __forceinline__ void refresh_body(const ElxChunk &c, uint32_t scalar_only) {
    typedef typename Elem<LD>::vec4 lvec;
    typedef typename Elem<LD>::scalar lscalar;
    if (!c.lowp_out) return;
    lscalar *out = reinterpret_cast<lscalar *>(c.lowp_out);
    const uint64_t n = c.n_alloc;
    const uint64_t pieces = (n + kRefreshPiece - 1) / kRefreshPiece;
    for (uint64_t piece = blockIdx.x; piece < pieces; piece += gridDim.x) {
        const uint64_t base = piece * kRefreshPiece;
        if (base + kRefreshPiece <= n && !scalar_only) {
            const __amdgpu_buffer_rsrc_t pr = tile_rsrc(c.master + base, kRefreshPiece * sizeof(float));
            const __amdgpu_buffer_rsrc_t lr = tile_rsrc(out + base, kRefreshPiece * sizeof(lscalar));
            f32x4 P[kRefreshUnroll];
#pragma unroll
            for (int u = 0; u < kRefreshUnroll; ++u)
                P[u] = TileIo<f32x4>::load(pr, (threadIdx.x + u * kRefreshThreads) * (uint32_t)sizeof(f32x4));
#pragma unroll
            for (int u = 0; u < kRefreshUnroll; ++u) {
                lvec L;
#pragma unroll
                for (int k = 0; k < kVec; ++k) L[k] = Elem<LD>::from_f32(P[u][k]);
                TileIo<lvec>::store(lr, (threadIdx.x + u * kRefreshThreads) * (uint32_t)sizeof(lvec), L);
            }
        } else {
            const uint64_t left = n - base;
            const uint32_t cnt = left < kRefreshPiece ? (uint32_t)left : kRefreshPiece;
            for (uint32_t i = threadIdx.x; i < cnt; i += kRefreshThreads) out[base + i] = Elem<LD>::from_f32(c.master[base + i]);
        }
    }
}

template <int LD>
__global__ __launch_bounds__(kRefreshThreads) void refresh_kernel(const ElxChunk *__restrict__ chunks,
                                                                  uint32_t scalar_only) {
    const ElxChunk c = chunks[blockIdx.y];
    refresh_body<LD>(c, scalar_only);
}

// One buffer, described in the kernel arguments: no table in device memory is needed.
template <int LD>
__global__ __launch_bounds__(kRefreshThreads) void refresh_one_kernel(ElxChunk c, uint32_t scalar_only) {
    refresh_body<LD>(c, scalar_only);
}

// ---------------------------------------------------------------------------------------------
// stats: overflow flag + sum of squares
// ---------------------------------------------------------------------------------------------

__device__ __forceinline__ double wave_sum(double x) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x += __shfl_down(x, off, 64);
    return x;
}

// Folds (sum, flag) over the workgroup; the result is valid in thread 0.  Fixed order.
__device__ __forceinline__ void block_fold(double &sum, uint32_t &flag) {
    __shared__ double s_sum[kStatsThreads / 64];
    __shared__ uint32_t s_flag[kStatsThreads / 64];
    sum = wave_sum(sum);
    flag = __ballot(flag != 0) != 0ull ? 1u : 0u;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) {
        s_sum[wave] = sum;
        s_flag[wave] = flag;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0.0;
        uint32_t f = 0;
        for (int w = 0; w < kStatsThreads / 64; ++w) {
            t += s_sum[w];
            f |= s_flag[w];
        }
        sum = t;
        flag = f;
    }
}

// x*x added in fp32; x*0 added into `poison`, which turns NaN exactly when x is inf or NaN.
__device__ __forceinline__ void stats_elem(float x, float &acc, float &poison) {
    acc = fmaf(x, x, acc);
    poison = fmaf(x, 0.0f, poison);
}

template <int GD, bool KEEP>
__device__ __forceinline__ void grad_stats_body(const ElxChunk &c, uint32_t bpc, ElxStats *__restrict__ partials,
                                                uint32_t scalar_only) {
    typedef typename Elem<GD>::scalar gscalar;
    constexpr uint32_t kEpl = 16 / sizeof(gscalar);    // elements per lane per 128-bit load
    constexpr uint32_t kSSpan = kStatsThreads * kEpl;
    constexpr uint32_t kSTile = kSSpan * kStatsUnroll;
    typedef gscalar gvec __attribute__((ext_vector_type(kEpl)));

    const gscalar *g = reinterpret_cast<const gscalar *>(c.grad);
    const uint64_t n = g ? c.n_valid : 0;
    const uint64_t n_tiles = (n + kSTile - 1) / kSTile;

    double sum = 0.0;
    float poison = 0.0f;
    for (uint64_t t = blockIdx.x; t < n_tiles; t += bpc) {
        const uint64_t base = t * kSTile;
        float acc = 0.0f;
        if (base + kSTile <= n && !scalar_only) {
            const gvec *gp = reinterpret_cast<const gvec *>(g + base) + threadIdx.x;
            gvec G[kStatsUnroll];
#pragma unroll
            for (int u = 0; u < kStatsUnroll; ++u) G[u] = ld_stream<KEEP>(gp + u * kStatsThreads);
#pragma unroll
            for (int u = 0; u < kStatsUnroll; ++u)
#pragma unroll
                for (uint32_t k = 0; k < kEpl; ++k) stats_elem(Elem<GD>::to_f32(G[u][k]), acc, poison);
        } else {
            const uint64_t left = n - base;
            const uint32_t tile_n = left < kSTile ? (uint32_t)left : kSTile;
            for (uint32_t i = threadIdx.x; i < tile_n; i += kStatsThreads)
                stats_elem(Elem<GD>::to_f32(g[base + i]), acc, poison);
        }
        sum += (double)acc;
    }
    uint32_t flag = (poison != poison) ? 1u : 0u;
    block_fold(sum, flag);
    if (threadIdx.x == 0) {
        ElxStats r;
        r.sumsq = sum;
        r.overflow = flag;
        r.reserved = 0;
        partials[(uint64_t)blockIdx.y * bpc + blockIdx.x] = r;
    }
}

template <int GD, bool KEEP>
__global__ __launch_bounds__(kStatsThreads) void grad_stats_kernel(const ElxChunk *__restrict__ chunks, uint32_t bpc,
                                                                   ElxStats *__restrict__ partials,
                                                                   uint32_t scalar_only) {
    const ElxChunk c = chunks[blockIdx.y];
    grad_stats_body<GD, KEEP>(c, bpc, partials, scalar_only);
}

// One buffer, described in the kernel arguments.
template <int GD>
__global__ __launch_bounds__(kStatsThreads) void grad_stats_one_kernel(ElxChunk c, uint32_t bpc,
                                                                       ElxStats *__restrict__ partials,
                                                                       uint32_t scalar_only) {
    grad_stats_body<GD, false>(c, bpc, partials, scalar_only);
}

__global__ __launch_bounds__(kStatsThreads) void stats_finish_kernel(const ElxStats *__restrict__ partials,
                                                                     uint32_t bpc, ElxStats *__restrict__ out) {
    const ElxStats *row = partials + (uint64_t)blockIdx.x * bpc;
    double sum = 0.0;
    uint32_t flag = 0;
    for (uint32_t i = threadIdx.x; i < bpc; i += kStatsThreads) {
        sum += row[i].sumsq;
        flag |= row[i].overflow;
    }
    block_fold(sum, flag);
    if (threadIdx.x == 0) {
        ElxStats r;
        r.sumsq = sum;
        r.overflow = flag;
        r.reserved = 0;
        out[blockIdx.x] = r;
    }
}

// ---------------------------------------------------------------------------------------------
// gradient landing: payload -> shard, with the stats riding the copy
// ---------------------------------------------------------------------------------------------

// dst[0, n_alloc) = cast(src * mul) for every row, and the stats of dst[0, n_valid) -- the values as
// they sit in the shard afterwards, which is what the flags of the reference are taken from.  A row
// uses `grad` as the source, `lowp_out` as the destination.  With MUL the product is first rounded
// to the source type (an in-place scaling of the payload), then cast.  Without MUL and with equal
// types the bits are moved untouched.
//
// A copy is a 1:1 read/write stream like the update, and wants the same shape: one wavefront per
// workgroup, one tile per workgroup (4 x 128-bit loads per lane: 4 KiB of source), residency capped
// through the LDS reservation, tiles handed out in address order by the dispatcher.  Grid
// (blocks_per_row, n_rows); when a row has more tiles than blocks a workgroup takes several
// (stride gridDim.x).  Every workgroup leaves one ElxStats partial, folded afterwards in a fixed
// order by stats_fold_kernel / stats_finish_kernel.
constexpr uint32_t kDefaultLandBlocksPerCu = 10;
constexpr uint32_t kDefaultLandBlocksPerCuNarrowing = 13;    // fp32 payload into a 16-bit shard: half the bytes go out
constexpr uint32_t kFoldBlocks = 64;           // first-stage workgroups per row when partials are many
constexpr uint32_t kFoldThreshold = 2048;      // partials per row above which the fold has two stages

template <int SD, int DD, bool MUL>
__device__ __forceinline__ typename Elem<DD>::scalar land_elem(typename Elem<SD>::scalar x, float mul, float &as_f32) {
    if constexpr (SD == DD && !MUL) {
        as_f32 = Elem<SD>::to_f32(x);
        return x;
    } else {
        float v = Elem<SD>::to_f32(x);
        if constexpr (MUL) {
            v = v * mul;
            // keep the product a plain fp32 multiply: folded into a mixed-precision fma with a +0
            // addend it would turn -0 * mul into +0
            asm volatile("" : "+v"(v));
            v = Elem<SD>::to_f32(Elem<SD>::from_f32(v));
        }
        const typename Elem<DD>::scalar d = Elem<DD>::from_f32(v);
        as_f32 = Elem<DD>::to_f32(d);
        return d;
    }
}

template <int BYTES>
struct LaneIo;
template <>
struct LaneIo<16> {
    typedef u32x4 raw;
    static __device__ __forceinline__ raw load(__amdgpu_buffer_rsrc_t r, uint32_t off) {
        return __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, kAuxLoad);
    }
    // KEEP: an ordinary store, which leaves the line in the memory-side cache for a launch that reads it soon
    template <bool KEEP>
    static __device__ __forceinline__ void store(__amdgpu_buffer_rsrc_t r, uint32_t off, raw x) {
        __builtin_amdgcn_raw_buffer_store_b128(x, r, (int)off, 0, KEEP ? 0 : kAuxStore);
    }
};
template <>
struct LaneIo<8> {
    typedef u32x2 raw;
    static __device__ __forceinline__ raw load(__amdgpu_buffer_rsrc_t r, uint32_t off) {
        return __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, kAuxLoad);
    }
    template <bool KEEP>
    static __device__ __forceinline__ void store(__amdgpu_buffer_rsrc_t r, uint32_t off, raw x) {
        __builtin_amdgcn_raw_buffer_store_b64(x, r, (int)off, 0, KEEP ? 0 : kAuxStore);
    }
};

template <int SD, int DD, bool MUL, bool KEEP>
__global__ __launch_bounds__(kWave) void land_grads_kernel(const ElxChunk *__restrict__ rows, float mul,
                                                           ElxStats *__restrict__ partials, uint32_t scalar_only) {
    typedef typename Elem<SD>::scalar sscalar;
    typedef typename Elem<DD>::scalar dscalar;
    constexpr uint32_t kEpl = 16 / sizeof(sscalar);              // elements per lane per 128-bit load
    constexpr uint32_t kLSpan = kWave * kEpl;
    constexpr uint32_t kLTile = kLSpan * kLandUnroll;
    constexpr int kDstBytes = (int)(kEpl * sizeof(dscalar));     // 16, or 8 for fp32 -> 16-bit
    typedef sscalar svec __attribute__((ext_vector_type(kEpl)));
    typedef dscalar dvec __attribute__((ext_vector_type(kEpl)));

    const ElxChunk c = load_chunk_row(rows + blockIdx.y);
    const sscalar *src = reinterpret_cast<const sscalar *>(c.grad);    // NULL: the source is all zeros
    dscalar *dst = reinterpret_cast<dscalar *>(c.lowp_out);
    const uint64_t n = dst ? c.n_alloc : 0;
    const uint64_t nv = c.n_valid < n ? c.n_valid : n;
    // 128-bit accesses need both ends of the row on a 16-byte boundary (tiles keep that alignment)
    const bool vec_ok = !scalar_only && ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) == 0;

    float acc = 0.0f, poison = 0.0f;
    double sum = 0.0;
    for (uint64_t base = (uint64_t)blockIdx.x * kLTile; base < n; base += (uint64_t)gridDim.x * kLTile) {
        if (base + kLTile <= n && vec_ok && (base + kLTile <= nv || base >= nv)) {
            // an empty resource returns zero for every lane: the NULL source without a branch
            const __amdgpu_buffer_rsrc_t sr = tile_rsrc(src ? src + base : nullptr, src ? kLTile * sizeof(sscalar) : 0u);
            const __amdgpu_buffer_rsrc_t dr = tile_rsrc(dst + base, kLTile * sizeof(dscalar));
            svec S[kLandUnroll];
#pragma unroll
            for (int u = 0; u < kLandUnroll; ++u)
                S[u] = __builtin_bit_cast(svec, LaneIo<16>::load(sr, (threadIdx.x + u * kWave) * 16u));
            float F[kLandUnroll][kEpl];
#pragma unroll
            for (int u = 0; u < kLandUnroll; ++u) {
                dvec D;
#pragma unroll
                for (uint32_t k = 0; k < kEpl; ++k) D[k] = land_elem<SD, DD, MUL>(S[u][k], mul, F[u][k]);
                LaneIo<kDstBytes>::template store<KEEP>(dr, (threadIdx.x + u * kWave) * (uint32_t)kDstBytes,
                                                        __builtin_bit_cast(typename LaneIo<kDstBytes>::raw, D));
            }
            if (base < nv) {    // wave-uniform: the tile lies inside the valid head
#pragma unroll
                for (int u = 0; u < kLandUnroll; ++u)
#pragma unroll
                    for (uint32_t k = 0; k < kEpl; ++k) stats_elem(F[u][k], acc, poison);
            }
        } else {
            const uint64_t left = n - base;
            const uint32_t tile_n = left < kLTile ? (uint32_t)left : kLTile;
            for (uint32_t i = threadIdx.x; i < tile_n; i += kWave) {
                float f;
                const sscalar x = src ? src[base + i] : sscalar(0);
                dst[base + i] = land_elem<SD, DD, MUL>(x, mul, f);
                if (base + i < nv) stats_elem(f, acc, poison);
            }
        }
        sum += (double)acc;
        acc = 0.0f;
    }
    sum = wave_sum(sum);
    const uint32_t flag = __ballot(poison != poison) != 0ull ? 1u : 0u;
    if (threadIdx.x == 0) {
        ElxStats r;
        r.sumsq = sum;
        r.overflow = flag;
        r.reserved = 0;
        partials[(uint64_t)blockIdx.y * gridDim.x + blockIdx.x] = r;
    }
}

// Folding the partials of a landing launch.  The partials are laid out [row][bpr]; the rows that
// feed one output record ("slot") are consecutive, so a slot owns one contiguous run of partials:
// rows [offsets[slot], offsets[slot + 1]) when an offsets table is given, row `slot` otherwise.
__device__ __forceinline__ void slot_range(const uint32_t *__restrict__ offsets, uint32_t slot, uint32_t bpr,
                                           uint64_t &begin, uint64_t &count) {
    const uint32_t r0 = offsets ? offsets[slot] : slot;
    const uint32_t r1 = offsets ? offsets[slot + 1] : slot + 1;
    begin = (uint64_t)r0 * bpr;
    count = (uint64_t)(r1 - r0) * bpr;
}

// First stage: workgroup j of slot y folds its contiguous share of the slot's partials into
// mid[y * gridDim.x + j].  Second stage: stats_finish_kernel over gridDim.x records per slot.
__global__ __launch_bounds__(kStatsThreads) void stats_fold_kernel(const ElxStats *__restrict__ partials, uint32_t bpr,
                                                                   const uint32_t *__restrict__ offsets,
                                                                   ElxStats *__restrict__ mid) {
    uint64_t begin, count;
    slot_range(offsets, blockIdx.y, bpr, begin, count);
    const uint64_t share = (count + gridDim.x - 1) / gridDim.x;
    const uint64_t lo = blockIdx.x * share;
    const uint64_t hi = lo + share < count ? lo + share : count;
    const ElxStats *run = partials + begin;
    double sum = 0.0;
    uint32_t flag = 0;
    for (uint64_t i = lo + threadIdx.x; i < hi; i += kStatsThreads) {
        sum += run[i].sumsq;
        flag |= run[i].overflow;
    }
    block_fold(sum, flag);
    if (threadIdx.x == 0) {
        ElxStats r;
        r.sumsq = sum;
        r.overflow = flag;
        r.reserved = 0;
        mid[(uint64_t)blockIdx.y * gridDim.x + blockIdx.x] = r;
    }
}

// ---------------------------------------------------------------------------------------------
// the decisions of the step, on the device
// ---------------------------------------------------------------------------------------------

__device__ __forceinline__ bool exact_reciprocal_dev(float s) {
    const uint32_t u = __builtin_bit_cast(uint32_t, s);
    const uint32_t exp = (u >> 23) & 0xFFu, man = u & 0x7FFFFFu;
    return (u >> 31) == 0 && man == 0 && exp >= 1 && exp <= 252;
}

// elixir/wrapper/optimizer.py:137-183 in the float64 arithmetic the host uses, one thread: any
// overflow -> skip; otherwise the combined scale = loss scale (x clip coefficient when the global
// norm exceeds max_norm).  Per chunk the squared norm passes through an fp32 norm
// (chunk.py:218-221), the sum over chunks through an fp32 buffer (optimizer.py:158-162).  The
// result goes into *out and into the gate words of every hyper record.
__device__ __forceinline__ ElxDecision finish_decision(uint32_t found, double norm_sqr, double loss_scale, double max_norm,
                                                       int clipping);

// `stats` may have been written by other workgroups of the same launch: read through agent-scope loads.
__device__ __forceinline__ ElxDecision decide_from_stats(const ElxStats *stats, uint32_t n, double loss_scale,
                                                         double max_norm, int clipping) {
    uint32_t found = 0;
    double norm_sqr = 0.0;
    for (uint32_t i = 0; i < n; ++i) {
        found |= __hip_atomic_load(&stats[i].overflow, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint64_t bits = __hip_atomic_load(reinterpret_cast<const uint64_t *>(&stats[i].sumsq), __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
        const float nrm = (float)sqrt(__builtin_bit_cast(double, bits));
        norm_sqr += (double)nrm * (double)nrm;
    }
    return finish_decision(found, norm_sqr, loss_scale, max_norm, clipping);
}

__device__ __forceinline__ ElxDecision finish_decision(uint32_t found, double norm_sqr, double loss_scale, double max_norm,
                                                       int clipping) {
    ElxDecision d;
    d.skip = found ? 1u : 0u;
    d.total_norm = 0.0;
    double combined = loss_scale;
    if (clipping) {
        d.total_norm = sqrt((double)(float)norm_sqr);
        const double clip = ((d.total_norm / loss_scale) + 1e-6) / max_norm;
        if (clip > 1.0) combined = clip * loss_scale;
    }
    if (combined == 1.0) combined = -1.0;
    d.combined_scale = combined;
    d.div_scale = (float)combined;
    d.inv_scale = 1.0f;
    d.mode = kDivNone;
    if (d.div_scale > 0.0f) {
        if (exact_reciprocal_dev(d.div_scale)) {
            d.mode = kDivMulInv;
            d.inv_scale = 1.0f / d.div_scale;
        } else {
            d.mode = kDivTrue;
        }
    }
    return d;
}

__global__ void decide_kernel(const ElxStats *__restrict__ stats, uint32_t n, double loss_scale, double max_norm,
                              int clipping, ElxHyper *__restrict__ hypers, uint32_t n_hypers,
                              ElxDecision *__restrict__ out) {
    if (blockIdx.x != 0 || threadIdx.x != 0) return;
    const ElxDecision d = decide_from_stats(stats, n, loss_scale, max_norm, clipping);
    *out = d;
    for (uint32_t i = 0; i < n_hypers; ++i) {
        hypers[i].gate_div_scale = d.div_scale;
        hypers[i].gate_inv_scale = d.inv_scale;
        hypers[i].gate = d.mode | (d.skip << 8);
    }
}

// The fold of the stats partials and the decisions of the step in ONE launch whose arguments never
// change from step to step (so that it can sit in a recorded graph): what does change -- loss scale,
// clipping threshold, the hyper records of the step -- is read from a control block in memory, which
// may be pinned host memory that the host rewrites before every step.
//
// Grid: one workgroup per chunk.  Workgroup b folds the partials of chunk b exactly as
// stats_finish_kernel does (same order, same bits) and publishes the record; the workgroup that
// finds every other one done (a counter, left at zero again for the next launch) decides: it copies
// the hyper records of the control block into the device table of the update launch with the gate
// words filled in, writes the decision, and reports to the host -- decision and per-chunk records
// first, the sequence number of the control block last, all with system-scope stores, so that a host
// polling the sequence number in pinned memory sees a complete report while the update launch that
// follows is still running.
constexpr uint32_t kMaxCtlHypers = 256;
constexpr uint32_t kCtlWords = (uint32_t)(sizeof(ElxStepCtl) + kMaxCtlHypers * sizeof(ElxHyper)) / 4u;
constexpr uint32_t kCtlEarlyHypers = 4;    // records fetched with the header, before anyone knows how many there are
static_assert((sizeof(ElxStepCtl) + kCtlEarlyHypers * sizeof(ElxHyper)) / 4u <= kStatsThreads, "one early load per thread");
constexpr uint32_t kDecideChunksInLds = 1024;    // per-chunk records staged in LDS for the decision loop

template <typename T>
__device__ __forceinline__ void store_system(T *p, T v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// The decision arithmetic of decide_from_stats over records staged in LDS.
__device__ __forceinline__ void accumulate_decision(double sumsq, uint32_t overflow, uint32_t &found, double &norm_sqr) {
    found |= overflow;
    const float nrm = (float)sqrt(sumsq);
    norm_sqr += (double)nrm * (double)nrm;
}

__device__ __forceinline__ double load_sumsq_agent(const ElxStats *r) {
    return __builtin_bit_cast(double, __hip_atomic_load(reinterpret_cast<const uint64_t *>(&r->sumsq), __ATOMIC_RELAXED,
                                                        __HIP_MEMORY_SCOPE_AGENT));
}

__device__ __forceinline__ uint32_t load_overflow_agent(const ElxStats *r) {
    return __hip_atomic_load(&r->overflow, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__global__ __launch_bounds__(kStatsThreads) void finish_decide_kernel(const ElxStats *__restrict__ partials, uint32_t bpc,
                                                                      ElxStats *stats, uint32_t n_chunks,
                                                                      const ElxStepCtl *ctl, ElxHyper *hypers,
                                                                      uint32_t max_hypers, ElxDecision *out,
                                                                      ElxStepReport *report, uint32_t *counter,
                                                                      const ElxChunk *__restrict__ rows,
                                                                      ElxChunk *__restrict__ gated_rows, uint32_t n_rows,
                                                                      uint32_t *armed) {
    __shared__ uint32_t s_last;
    __shared__ __align__(16) uint32_t s_ctl[kCtlWords];
    __shared__ ElxDecision s_decision;
    __shared__ ElxStats s_stats[kDecideChunksInLds];
    // Every workgroup asks for the head of the control block at once (it may sit in host memory, a long
    // way off): the answer travels while the partials are folded, and the workgroup that ends up deciding
    // has it at hand.  System-scope loads: the host rewrites the block between launches.
    // Never beyond the max_hypers records the caller vouches for behind the header.
    const uint32_t *cw = reinterpret_cast<const uint32_t *>(ctl);
    const uint32_t early_words =
        (uint32_t)(sizeof(ElxStepCtl) + (max_hypers < kCtlEarlyHypers ? max_hypers : kCtlEarlyHypers) * sizeof(ElxHyper)) / 4u;
    uint32_t early = 0;
    if (threadIdx.x < early_words) early = __hip_atomic_load(cw + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    {
        const ElxStats *row = partials + (uint64_t)blockIdx.x * bpc;
        double sum = 0.0;
        uint32_t flag = 0;
        for (uint32_t i = threadIdx.x; i < bpc; i += kStatsThreads) {
            sum += row[i].sumsq;
            flag |= row[i].overflow;
        }
        block_fold(sum, flag);
        if (threadIdx.x == 0) {
            __hip_atomic_store(reinterpret_cast<uint64_t *>(&stats[blockIdx.x].sumsq), __builtin_bit_cast(uint64_t, sum),
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&stats[blockIdx.x].overflow, flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&stats[blockIdx.x].reserved, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // release the record, then count this workgroup as done; the one that completes the count decides
            const uint32_t done = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
            s_last = done == n_chunks - 1 ? 1u : 0u;
        }
    }
    if (threadIdx.x < early_words) s_ctl[threadIdx.x] = early;
    __syncthreads();
    if (!s_last) return;

    // ---- the last workgroup decides
    const ElxStepCtl *c = reinterpret_cast<const ElxStepCtl *>(s_ctl);
    const uint32_t cap = max_hypers < kMaxCtlHypers ? max_hypers : kMaxCtlHypers;
    const bool valid = c->loss_scale > 0.0 && (!c->clipping || c->max_norm > 0.0) && c->n_hypers <= cap;
    const uint32_t n_hypers = valid ? c->n_hypers : 0u;
    // the hyper records behind the ones that came with the header, and every chunk's record, side by side
    for (uint32_t i = early_words + threadIdx.x; i < (sizeof(ElxStepCtl) + n_hypers * sizeof(ElxHyper)) / 4u;
         i += kStatsThreads)
        s_ctl[i] = __hip_atomic_load(cw + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    const uint32_t staged = n_chunks < kDecideChunksInLds ? n_chunks : kDecideChunksInLds;
    for (uint32_t i = threadIdx.x; i < staged; i += kStatsThreads) {
        s_stats[i].sumsq = load_sumsq_agent(stats + i);
        s_stats[i].overflow = load_overflow_agent(stats + i);
        s_stats[i].reserved = 0;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        // decide_from_stats, in the same order: over the staged records, then over whatever did not fit
        uint32_t found = 0;
        double norm_sqr = 0.0;
        for (uint32_t i = 0; i < staged; ++i) accumulate_decision(s_stats[i].sumsq, s_stats[i].overflow, found, norm_sqr);
        for (uint32_t i = staged; i < n_chunks; ++i)
            accumulate_decision(load_sumsq_agent(stats + i), load_overflow_agent(stats + i), found, norm_sqr);
        ElxDecision d = finish_decision(found, norm_sqr, valid ? c->loss_scale : 1.0, valid ? c->max_norm : 1.0,
                                        valid ? (int)c->clipping : 0);
        if (!valid) d.skip = 1u;    // an unusable control block: nothing is updated, and the report says why
        s_decision = d;
        *out = d;
    }
    __syncthreads();
    const ElxDecision d = s_decision;
    // the hyper table of the update launch: the step's records with the gate words of this decision.  When
    // the control block is unusable every record the table can hold gets the skip gate.
    // (word by word: nine words of the step's record, or zeros, then the three gate words)
    constexpr uint32_t kHyperWords = sizeof(ElxHyper) / 4u, kGateWord = offsetof(ElxHyper, gate_div_scale) / 4u;
    static_assert(kHyperWords == kGateWord + 3 && offsetof(ElxHyper, gate) / 4u == kGateWord + 2, "gate words come last");
    const uint32_t *src = s_ctl + sizeof(ElxStepCtl) / 4u;
    uint32_t *dst = reinterpret_cast<uint32_t *>(hypers);
    const uint32_t gate_words[3] = {__builtin_bit_cast(uint32_t, d.div_scale), __builtin_bit_cast(uint32_t, d.inv_scale),
                                    d.mode | (d.skip << 8)};
    for (uint32_t i = threadIdx.x; i < (valid ? n_hypers : max_hypers) * kHyperWords; i += kStatsThreads) {
        const uint32_t word = i % kHyperWords;
        uint32_t value = valid ? src[i] : 0u;
        if (word == kGateWord) value = gate_words[0];
        if (word == kGateWord + 1) value = gate_words[1];
        if (word == kGateWord + 2) value = gate_words[2];
        dst[i] = value;
    }
    // The row table of the gated update launch, when the caller keeps one for it: no row has a valid element
    // when the step is skipped, every row has its own count back afterwards.  A row without valid elements only
    // has its low-precision copy refreshed, and the update launch learns that from the record it fetches first
    // of all: a skipped step then moves 6 bytes per element instead of 16, and an ordinary step pays nothing
    // for it (asking for the skip flag itself at the top of the update kernel cost every step 3.6 %).  *armed
    // says whether the table holds zeros now, so that the ordinary step after an ordinary step writes nothing.
    if (gated_rows) {
        const uint32_t was_armed = __hip_atomic_load(armed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (d.skip || was_armed) {
            for (uint32_t i = threadIdx.x; i < n_rows; i += kStatsThreads) gated_rows[i].n_valid = d.skip ? 0ull : rows[i].n_valid;
            __syncthreads();
            if (threadIdx.x == 0) __hip_atomic_store(armed, d.skip ? 1u : 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (report) {
        const uint32_t *dw = reinterpret_cast<const uint32_t *>(&s_decision);
        uint32_t *rw = reinterpret_cast<uint32_t *>(&report->decision);
        for (uint32_t i = threadIdx.x; i < sizeof(ElxDecision) / 4u; i += kStatsThreads) store_system(rw + i, dw[i]);
        ElxStats *rs = reinterpret_cast<ElxStats *>(report + 1);
        for (uint32_t i = threadIdx.x; i < n_chunks; i += kStatsThreads) {
            const double sumsq = i < staged ? s_stats[i].sumsq : load_sumsq_agent(stats + i);
            const uint32_t overflow = i < staged ? s_stats[i].overflow : load_overflow_agent(stats + i);
            store_system(reinterpret_cast<uint64_t *>(&rs[i].sumsq), __builtin_bit_cast(uint64_t, sumsq));
            store_system(&rs[i].overflow, overflow);
            store_system(&rs[i].reserved, 0u);
        }
        if (threadIdx.x == 0) {
            store_system(&report->n_chunks, n_chunks);
            store_system(&report->status, valid ? 0 : (int32_t)ELX_E_RANGE);
        }
        __threadfence_system();
        __syncthreads();
        if (threadIdx.x == 0)
            __hip_atomic_store(&report->seq, c->seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    if (threadIdx.x == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Hyper records from the kernel arguments into the device table of an update launch: a handful of
// records reach the device inside the launch packet itself, without a staging buffer and a copy to
// order and to keep alive.
__global__ __launch_bounds__(kWave) void put_hypers_kernel(HyperPack pack, uint32_t n_words, uint32_t *__restrict__ dst) {
    // the pack is read where it lies, in the argument segment (indexing a by-value aggregate with the lane
    // number would copy it to private memory first)
    typedef const uint32_t __attribute__((address_space(4))) *kernarg_words;
    kernarg_words src = (kernarg_words)__builtin_amdgcn_kernarg_segment_ptr();
    for (uint32_t i = threadIdx.x; i < n_words; i += kWave) dst[i] = src[i];
}

// ---------------------------------------------------------------------------------------------
// host side of the ABI
// ---------------------------------------------------------------------------------------------

// flag bits an update launch understands
constexpr uint32_t kUpdateFlags = ELX_FLAG_SCALAR_ONLY | ELX_FLAG_KEEP_CACHED | ELX_FLAG_KEEP_STATE_CACHED;

// The cache policy the flags of an update launch ask for.  Without a low-precision copy kKeepLowp has nothing
// to act on and is the streaming launch.
template <int LD>
int policy_of(uint32_t flags) {
    if (flags & ELX_FLAG_KEEP_STATE_CACHED) return kKeepState;
    if ((flags & ELX_FLAG_KEEP_CACHED) && LD != ELX_NONE) return kKeepLowp;
    return kStream;
}

template <int GD, int LD, bool GATED>
int launch_step_policy(uint32_t lds, hipStream_t st, const ElxChunk *chunks, uint32_t n_chunks, const ElxSeg *segs,
                       const ElxHyper *hypers, uint32_t grid_tiles, Unscale us, uint32_t flags, uint32_t scalar_only) {
    const dim3 grid(grid_tiles, n_chunks);
    constexpr int kLowp = LD != ELX_NONE ? kKeepLowp : kStream;    // no third instantiation without a low-precision copy
    switch (policy_of<LD>(flags)) {
        case kKeepState:
            hipLaunchKernelGGL((adam_step_kernel<GD, LD, GATED, kKeepState>), grid, dim3(kWave), lds, st, chunks, segs, hypers,
                               us, scalar_only);
            break;
        case kKeepLowp:
            hipLaunchKernelGGL((adam_step_kernel<GD, LD, GATED, kLowp>), grid, dim3(kWave), lds, st, chunks, segs, hypers, us,
                               scalar_only);
            break;
        default:
            hipLaunchKernelGGL((adam_step_kernel<GD, LD, GATED, kStream>), grid, dim3(kWave), lds, st, chunks, segs, hypers, us,
                               scalar_only);
    }
    return (int)hipGetLastError();
}

template <int GD, int LD>
int launch_step(uint32_t lds, hipStream_t st, const ElxChunk *chunks, uint32_t n_chunks, const ElxSeg *segs,
                const ElxHyper *hypers, uint32_t grid_tiles, Unscale us, bool gated, uint32_t flags, uint32_t scalar_only) {
    if (gated)
        return launch_step_policy<GD, LD, true>(lds, st, chunks, n_chunks, segs, hypers, grid_tiles, us, flags, scalar_only);
    return launch_step_policy<GD, LD, false>(lds, st, chunks, n_chunks, segs, hypers, grid_tiles, us, flags, scalar_only);
}

int dispatch_step(int gd, int ld, uint32_t lds, hipStream_t st, const ElxChunk *chunks, uint32_t n_chunks,
                  const ElxSeg *segs, const ElxHyper *hypers, uint32_t grid_tiles, Unscale us, bool gated, uint32_t flags,
                  uint32_t scalar_only) {
#define ELX_CASE(G, L)                                                                                   \
    if (gd == G && ld == L)                                                                              \
        return launch_step<G, L>(lds, st, chunks, n_chunks, segs, hypers, grid_tiles, us, gated, flags, scalar_only);
    ELX_CASE(ELX_F32, ELX_NONE)
    ELX_CASE(ELX_F32, ELX_F32)
    ELX_CASE(ELX_F16, ELX_NONE)
    ELX_CASE(ELX_F16, ELX_F16)
    ELX_CASE(ELX_BF16, ELX_NONE)
    ELX_CASE(ELX_BF16, ELX_BF16)
#undef ELX_CASE
    return ELX_E_DTYPE;
}

template <int GD, int LD>
int launch_step_args(uint32_t lds, hipStream_t st, const HyperPack &pack, const ElxChunk *chunks, uint32_t n_chunks,
                     const ElxSeg *segs, uint32_t grid_tiles, Unscale us, uint32_t flags, uint32_t scalar_only) {
    const dim3 grid(grid_tiles, n_chunks);
    constexpr int kLowp = LD != ELX_NONE ? kKeepLowp : kStream;
    switch (policy_of<LD>(flags)) {
        case kKeepState:
            hipLaunchKernelGGL((adam_step_args_kernel<GD, LD, kKeepState>), grid, dim3(kWave), lds, st, pack, chunks, segs, us,
                               scalar_only);
            break;
        case kKeepLowp:
            hipLaunchKernelGGL((adam_step_args_kernel<GD, LD, kLowp>), grid, dim3(kWave), lds, st, pack, chunks, segs, us,
                               scalar_only);
            break;
        default:
            hipLaunchKernelGGL((adam_step_args_kernel<GD, LD, kStream>), grid, dim3(kWave), lds, st, pack, chunks, segs, us,
                               scalar_only);
    }
    return (int)hipGetLastError();
}

int dispatch_step_args(int gd, int ld, uint32_t lds, hipStream_t st, const HyperPack &pack, const ElxChunk *chunks,
                       uint32_t n_chunks, const ElxSeg *segs, uint32_t grid_tiles, Unscale us, uint32_t flags,
                       uint32_t scalar_only) {
#define ELX_CASE(G, L)                                                                                   \
    if (gd == G && ld == L)                                                                              \
        return launch_step_args<G, L>(lds, st, pack, chunks, n_chunks, segs, grid_tiles, us, flags, scalar_only);
    ELX_CASE(ELX_F32, ELX_NONE)
    ELX_CASE(ELX_F32, ELX_F32)
    ELX_CASE(ELX_F16, ELX_NONE)
    ELX_CASE(ELX_F16, ELX_F16)
    ELX_CASE(ELX_BF16, ELX_NONE)
    ELX_CASE(ELX_BF16, ELX_BF16)
#undef ELX_CASE
    return ELX_E_DTYPE;
}

// Device address of `scratch` on the current device, looked up once per device (each GPU holds its own
// copy of the array at its own address).
constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];

// `stream` (NULL: the default stream) is the one the caller's launches will go to.  Refused with
// ELX_E_STATE: a stream that belongs to another GPU than the calling thread's current one (the array's
// address is only good there), and a first call on a device made while the stream is capturing (the
// address lookup is not something to do inside a capture).
int scratch_of_current_device(hipStream_t stream, void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return ELX_E_SIZE;
    if (stream) {
        hipDevice_t of_stream, current;
        if (hipStreamGetDevice(stream, &of_stream) == hipSuccess && hipDeviceGet(&current, dev) == hipSuccess) {
            if (of_stream != current) return ELX_E_STATE;
        } else {
            (void)hipGetLastError();    // the query is a courtesy: a runtime that cannot answer leaves the rule to the caller
        }
    }
    void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) (void)hipGetLastError();
        if (capturing != hipStreamCaptureStatusNone) return ELX_E_STATE;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!ptr) return ELX_E_NULL;
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);    // two threads racing here store the same address
    }
    *out = ptr;
    return 0;
}

}    // namespace

template <int S, int D>
static int launch_land(bool scaled, bool keep, dim3 grid, uint32_t lds, hipStream_t st, const ElxChunk *d_rows, float mul,
                       ElxStats *d_partials, uint32_t scalar_only) {
    const dim3 block(kWave);
    if (scaled && keep)
        hipLaunchKernelGGL((land_grads_kernel<S, D, true, true>), grid, block, lds, st, d_rows, mul, d_partials, scalar_only);
    else if (scaled)
        hipLaunchKernelGGL((land_grads_kernel<S, D, true, false>), grid, block, lds, st, d_rows, mul, d_partials, scalar_only);
    else if (keep)
        hipLaunchKernelGGL((land_grads_kernel<S, D, false, true>), grid, block, lds, st, d_rows, mul, d_partials, scalar_only);
    else
        hipLaunchKernelGGL((land_grads_kernel<S, D, false, false>), grid, block, lds, st, d_rows, mul, d_partials, scalar_only);
    return (int)hipGetLastError();
}

template <int GD>
static void launch_grad_stats(bool keep, dim3 grid, hipStream_t st, const ElxChunk *d_chunks, uint32_t bpc,
                              ElxStats *d_partials, uint32_t scalar_only) {
    if (keep) {
        hipLaunchKernelGGL((grad_stats_kernel<GD, true>), grid, dim3(kStatsThreads), 0, st, d_chunks, bpc, d_partials,
                           scalar_only);
    } else {
        // A set that streams from HBM is read fastest with a shallow queue, like the update's streams: three
        // workgroups (twelve wavefronts, 48 KiB of loads in flight) per compute unit instead of the eight that
        // fit, held there by an LDS reservation no thread touches (-3.5 % on 2.6 and 13.5 GB of gradients;
        // a set served from the cache wants all eight).
        // (the kernel's own few bytes of static LDS come on top of the reservation: leave room for them, or
        // only two workgroups fit and the pass slows down by a fifth)
        const uint32_t lds = (kLdsPerCu / kStatsStreamBlocksPerCu - 1024u) & ~255u;
        hipLaunchKernelGGL((grad_stats_kernel<GD, false>), grid, dim3(kStatsThreads), lds, st, d_chunks, bpc, d_partials,
                           scalar_only);
    }
}

extern "C" {

int elx_version(void) { return ELX_ABI_VERSION; }

uint32_t elx_sizeof_chunk(void) { return (uint32_t)sizeof(ElxChunk); }
uint32_t elx_sizeof_seg(void) { return (uint32_t)sizeof(ElxSeg); }
uint32_t elx_sizeof_hyper(void) { return (uint32_t)sizeof(ElxHyper); }
uint32_t elx_sizeof_stats(void) { return (uint32_t)sizeof(ElxStats); }
uint32_t elx_sizeof_decision(void) { return (uint32_t)sizeof(ElxDecision); }

const char *elx_strerror(int code) {
    switch (code) {
        case 0: return "success";
        case ELX_E_NULL: return "elx: a required pointer is NULL";
        case ELX_E_DTYPE: return "elx: unknown or unsupported dtype combination";
        case ELX_E_ALIGN: return "elx: a chunk base pointer is not aligned to its element size";
        case ELX_E_RANGE: return "elx: a range is out of bounds (begin >= end, end > n_valid, n_valid > n_alloc, segment range or hyper index)";
        case ELX_E_ORDER: return "elx: segments of a chunk are not sorted or overlap";
        case ELX_E_TILES: return "elx: tile_begin / total_tiles disagree with the chunk sizes";
        case ELX_E_SIZE: return "elx: a count is zero, out of its allowed range, or exceeds what a launch can address";
        case ELX_E_STATE: return "elx: the call cannot be made in this state (a stream of another GPU than the current one, or a first call on a device made under stream capture)";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "elx: unknown error code";
}

int elx_grad_partials_mt(const ElxChunk *d_chunks, uint32_t n_chunks, int grad_dtype, uint32_t blocks_per_chunk,
                         ElxStats *d_partials, int flags, void *stream);

int elx_grad_stats_mt(const ElxChunk *d_chunks, uint32_t n_chunks, int grad_dtype, uint32_t blocks_per_chunk,
                      ElxStats *d_partials, ElxStats *d_stats, int flags, void *stream) {
    if (!d_stats) return ELX_E_NULL;
    if (int rc = elx_grad_partials_mt(d_chunks, n_chunks, grad_dtype, blocks_per_chunk, d_partials, flags, stream))
        return rc;
    hipLaunchKernelGGL(stats_finish_kernel, dim3(n_chunks), dim3(kStatsThreads), 0, (hipStream_t)stream, d_partials,
                       blocks_per_chunk, d_stats);
    return (int)hipGetLastError();
}

int elx_grad_partials_mt(const ElxChunk *d_chunks, uint32_t n_chunks, int grad_dtype, uint32_t blocks_per_chunk,
                         ElxStats *d_partials, int flags, void *stream) {
    if (!d_chunks || !d_partials) return ELX_E_NULL;
    if (n_chunks == 0 || n_chunks > 65535u || blocks_per_chunk == 0 || blocks_per_chunk > kMaxStatsBlocks)
        return ELX_E_SIZE;
    if ((uint32_t)flags & ~(uint32_t)(ELX_FLAG_SCALAR_ONLY | ELX_FLAG_KEEP_CACHED)) return ELX_E_RANGE;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid(blocks_per_chunk, n_chunks);
    const uint32_t so = ((uint32_t)flags & ELX_FLAG_SCALAR_ONLY) ? 1u : 0u;
    const bool keep = ((uint32_t)flags & ELX_FLAG_KEEP_CACHED) != 0;
    switch (grad_dtype) {
        case ELX_F32: launch_grad_stats<ELX_F32>(keep, grid, st, d_chunks, blocks_per_chunk, d_partials, so); break;
        case ELX_F16: launch_grad_stats<ELX_F16>(keep, grid, st, d_chunks, blocks_per_chunk, d_partials, so); break;
        case ELX_BF16: launch_grad_stats<ELX_BF16>(keep, grid, st, d_chunks, blocks_per_chunk, d_partials, so); break;
        default: return ELX_E_DTYPE;
    }
    return (int)hipGetLastError();
}

int elx_finish_decide_rows(const ElxStats *d_partials, uint32_t n_chunks, uint32_t blocks_per_chunk, ElxStats *d_stats,
                           const ElxStepCtl *ctl, ElxHyper *d_hypers, uint32_t max_hypers, ElxDecision *d_decision,
                           ElxStepReport *report, uint32_t *d_counter, const ElxChunk *d_rows, ElxChunk *d_gated_rows,
                           uint32_t n_rows, uint32_t *d_armed, void *stream) {
    if (!d_partials || !d_stats || !ctl || !d_decision || !d_counter || (max_hypers && !d_hypers)) return ELX_E_NULL;
    if (n_chunks == 0 || n_chunks > 65535u || blocks_per_chunk == 0 || blocks_per_chunk > kMaxLandBlocks ||
        max_hypers > kMaxCtlHypers)
        return ELX_E_SIZE;
    if (((uintptr_t)ctl | (uintptr_t)report | (uintptr_t)d_stats | (uintptr_t)d_decision) & 7u) return ELX_E_ALIGN;
    if (d_gated_rows) {
        if (!d_rows || !d_armed) return ELX_E_NULL;
        if (n_rows == 0 || n_rows > 65535u) return ELX_E_SIZE;
        if (d_rows == d_gated_rows) return ELX_E_RANGE;    // the counts are taken from a table nobody writes
        if ((((uintptr_t)d_rows | (uintptr_t)d_gated_rows) & 7u) || ((uintptr_t)d_armed & 3u)) return ELX_E_ALIGN;
    }
    hipLaunchKernelGGL(finish_decide_kernel, dim3(n_chunks), dim3(kStatsThreads), 0, (hipStream_t)stream, d_partials,
                       blocks_per_chunk, d_stats, n_chunks, ctl, d_hypers, max_hypers, d_decision, report, d_counter, d_rows,
                       d_gated_rows, d_gated_rows ? n_rows : 0u, d_armed);
    return (int)hipGetLastError();
}

int elx_finish_decide(const ElxStats *d_partials, uint32_t n_chunks, uint32_t blocks_per_chunk, ElxStats *d_stats,
                      const ElxStepCtl *ctl, ElxHyper *d_hypers, uint32_t max_hypers, ElxDecision *d_decision,
                      ElxStepReport *report, uint32_t *d_counter, void *stream) {
    return elx_finish_decide_rows(d_partials, n_chunks, blocks_per_chunk, d_stats, ctl, d_hypers, max_hypers, d_decision,
                                  report, d_counter, nullptr, nullptr, 0, nullptr, stream);
}

int elx_put_hypers(const ElxHyper *h_hypers, uint32_t n_hypers, ElxHyper *d_hypers, void *stream) {
    if (!h_hypers || !d_hypers) return ELX_E_NULL;
    if (n_hypers == 0) return ELX_E_SIZE;
    if ((uintptr_t)d_hypers & 3u) return ELX_E_ALIGN;
    for (uint32_t at = 0; at < n_hypers; at += kMaxArgHypers) {
        const uint32_t n = n_hypers - at < kMaxArgHypers ? n_hypers - at : kMaxArgHypers;
        HyperPack pack = {};
        __builtin_memcpy(pack.h, h_hypers + at, n * sizeof(ElxHyper));
        hipLaunchKernelGGL(put_hypers_kernel, dim3(1), dim3(kWave), 0, (hipStream_t)stream, pack,
                           n * (uint32_t)(sizeof(ElxHyper) / 4u), reinterpret_cast<uint32_t *>(d_hypers + at));
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return (int)e;
    }
    return 0;
}

uint32_t elx_sizeof_step_ctl(void) { return (uint32_t)sizeof(ElxStepCtl); }
uint32_t elx_sizeof_step_report(void) { return (uint32_t)sizeof(ElxStepReport); }
uint32_t elx_max_ctl_hypers(void) { return kMaxCtlHypers; }

uint32_t elx_static_partials(void) { return kStaticPartials; }

int elx_grad_stats_mt_static(const ElxChunk *d_chunks, uint32_t n_chunks, int grad_dtype, uint32_t blocks_per_chunk,
                             ElxStats *d_stats, int flags, void *stream) {
    if (!d_chunks || !d_stats) return ELX_E_NULL;
    if (n_chunks == 0 || n_chunks > 65535u || blocks_per_chunk == 0 || blocks_per_chunk > kMaxStatsBlocks)
        return ELX_E_SIZE;
    if ((uint64_t)n_chunks * blocks_per_chunk > kStaticPartials) return ELX_E_SIZE;
    if (!is_lowp_or_f32(grad_dtype)) return ELX_E_DTYPE;
    if ((uint32_t)flags & ~(uint32_t)(ELX_FLAG_SCALAR_ONLY | ELX_FLAG_KEEP_CACHED)) return ELX_E_RANGE;
    void *partials = nullptr;
    if (int rc = scratch_of_current_device((hipStream_t)stream, &partials)) return rc;
    // every partial the finish launch reads is written by the stats launch first: nothing to clear
    return elx_grad_stats_mt(d_chunks, n_chunks, grad_dtype, blocks_per_chunk, reinterpret_cast<ElxStats *>(partials),
                             d_stats, flags, stream);
}

int elx_adam_step_mt(const ElxChunk *d_chunks, uint32_t n_chunks, const ElxSeg *d_segs, uint32_t n_segs,
                     const ElxHyper *d_hypers, uint32_t n_hypers, uint64_t total_tiles, uint32_t grid_tiles_per_chunk,
                     float div_scale, int grad_dtype, int lowp_dtype, uint32_t flags, uint32_t blocks_per_cu,
                     void *stream) {
    if (!d_chunks || (n_segs && (!d_segs || !d_hypers))) return ELX_E_NULL;
    if (n_chunks == 0 || n_chunks > 65535u || total_tiles == 0 || total_tiles > 0x7FFFFFFFull || (n_segs && n_hypers == 0))
        return ELX_E_SIZE;
    if (grid_tiles_per_chunk == 0 || (uint64_t)grid_tiles_per_chunk * n_chunks < total_tiles) return ELX_E_TILES;
    if (!is_lowp_or_f32(grad_dtype)) return ELX_E_DTYPE;
    if (lowp_dtype != ELX_NONE && lowp_dtype != grad_dtype) return ELX_E_DTYPE;
    if (flags & ~kUpdateFlags) return ELX_E_RANGE;
    uint32_t lds = 0;
    if (int rc = occupancy_reservation(blocks_per_cu, &lds, grad_dtype == ELX_F32 ? kDefaultBlocksPerCu : kDefaultBlocksPerCuLowp))
        return rc;
    return dispatch_step(grad_dtype, lowp_dtype, lds, (hipStream_t)stream, d_chunks, n_chunks, d_segs, d_hypers,
                         grid_tiles_per_chunk, unscale_of(div_scale), false, flags,
                         (flags & ELX_FLAG_SCALAR_ONLY) ? 1u : 0u);
}

int elx_put_hypers(const ElxHyper *h_hypers, uint32_t n_hypers, ElxHyper *d_hypers, void *stream);

int elx_adam_step_put_mt(const ElxChunk *d_chunks, uint32_t n_chunks, const ElxSeg *d_segs, uint32_t n_segs,
                         const ElxHyper *h_hypers, ElxHyper *d_hypers, uint32_t n_hypers, uint64_t total_tiles,
                         uint32_t grid_tiles_per_chunk, float div_scale, int grad_dtype, int lowp_dtype, uint32_t flags,
                         uint32_t blocks_per_cu, void *stream) {
    if (!h_hypers || !d_hypers) return ELX_E_NULL;
    // every argument check of the update launch first: nothing goes out when the update would be refused
    if (!d_chunks || (n_segs && !d_segs)) return ELX_E_NULL;
    if (n_chunks == 0 || n_chunks > 65535u || total_tiles == 0 || total_tiles > 0x7FFFFFFFull || n_hypers == 0)
        return ELX_E_SIZE;
    if (grid_tiles_per_chunk == 0 || (uint64_t)grid_tiles_per_chunk * n_chunks < total_tiles) return ELX_E_TILES;
    if (!is_lowp_or_f32(grad_dtype)) return ELX_E_DTYPE;
    if (lowp_dtype != ELX_NONE && lowp_dtype != grad_dtype) return ELX_E_DTYPE;
    if (flags & ~kUpdateFlags) return ELX_E_RANGE;
    uint32_t lds = 0;
    if (int rc = occupancy_reservation(blocks_per_cu, &lds, grad_dtype == ELX_F32 ? kDefaultBlocksPerCu : kDefaultBlocksPerCuLowp))
        return rc;
    if (n_hypers <= kMaxArgHypers) {    // the records ride the update launch itself; d_hypers is not written
        HyperPack pack = {};
        __builtin_memcpy(pack.h, h_hypers, n_hypers * sizeof(ElxHyper));
        return dispatch_step_args(grad_dtype, lowp_dtype, lds, (hipStream_t)stream, pack, d_chunks, n_chunks, d_segs,
                                  grid_tiles_per_chunk, unscale_of(div_scale), flags,
                                  (flags & ELX_FLAG_SCALAR_ONLY) ? 1u : 0u);
    }
    if (int rc = elx_put_hypers(h_hypers, n_hypers, d_hypers, stream)) return rc;
    return elx_adam_step_mt(d_chunks, n_chunks, d_segs, n_segs, d_hypers, n_hypers, total_tiles, grid_tiles_per_chunk,
                            div_scale, grad_dtype, lowp_dtype, flags, blocks_per_cu, stream);
}

int elx_decide(const ElxStats *d_stats, uint32_t n_chunks, double loss_scale, double max_norm, int clipping,
               ElxHyper *d_hypers, uint32_t n_hypers, ElxDecision *d_decision, void *stream) {
    if (!d_stats || !d_decision || (n_hypers && !d_hypers)) return ELX_E_NULL;
    if (n_chunks == 0) return ELX_E_SIZE;
    if (!(loss_scale > 0.0) || (clipping && !(max_norm > 0.0))) return ELX_E_RANGE;
    hipLaunchKernelGGL(decide_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, d_stats, n_chunks, loss_scale, max_norm,
                       clipping, d_hypers, n_hypers, d_decision);
    return (int)hipGetLastError();
}

int elx_adam_step_gated_mt(const ElxChunk *d_chunks, uint32_t n_chunks, const ElxSeg *d_segs, uint32_t n_segs,
                           const ElxHyper *d_hypers, uint32_t n_hypers, uint64_t total_tiles,
                           uint32_t grid_tiles_per_chunk, int grad_dtype, int lowp_dtype, uint32_t flags,
                           uint32_t blocks_per_cu, void *stream) {
    if (!d_chunks || (n_segs && (!d_segs || !d_hypers))) return ELX_E_NULL;
    if (n_chunks == 0 || n_chunks > 65535u || total_tiles == 0 || total_tiles > 0x7FFFFFFFull || (n_segs && n_hypers == 0))
        return ELX_E_SIZE;
    if (grid_tiles_per_chunk == 0 || (uint64_t)grid_tiles_per_chunk * n_chunks < total_tiles) return ELX_E_TILES;
    if (!is_lowp_or_f32(grad_dtype)) return ELX_E_DTYPE;
    if (lowp_dtype != ELX_NONE && lowp_dtype != grad_dtype) return ELX_E_DTYPE;
    if (flags & ~kUpdateFlags) return ELX_E_RANGE;
    uint32_t lds = 0;
    if (int rc = occupancy_reservation(blocks_per_cu, &lds, grad_dtype == ELX_F32 ? kDefaultBlocksPerCu : kDefaultBlocksPerCuLowp))
        return rc;
    Unscale us;
    us.div_scale = -1.0f;
    us.inv_scale = 1.0f;
    us.mode = kDivNone;
    return dispatch_step(grad_dtype, lowp_dtype, lds, (hipStream_t)stream, d_chunks, n_chunks, d_segs, d_hypers,
                         grid_tiles_per_chunk, us, true, flags,
                         (flags & ELX_FLAG_SCALAR_ONLY) ? 1u : 0u);
}

int elx_writeback_mt(const ElxChunk *d_chunks, uint32_t n_chunks, int lowp_dtype, uint32_t blocks_per_chunk,
                     uint32_t flags, void *stream) {
    if (!d_chunks) return ELX_E_NULL;
    if (n_chunks == 0 || n_chunks > 65535u || blocks_per_chunk == 0 || blocks_per_chunk > kMaxRefreshBlocks) return ELX_E_SIZE;
    const dim3 grid(blocks_per_chunk, n_chunks);
    const uint32_t so = (flags & ELX_FLAG_SCALAR_ONLY) ? 1u : 0u;
    hipStream_t st = (hipStream_t)stream;
    uint32_t lds = 0;
    if (int rc = occupancy_reservation(kRefreshBlocksPerCu, &lds)) return rc;
    switch (lowp_dtype) {
        case ELX_F32: hipLaunchKernelGGL((refresh_kernel<ELX_F32>), grid, dim3(kRefreshThreads), lds, st, d_chunks, so); break;
        case ELX_F16: hipLaunchKernelGGL((refresh_kernel<ELX_F16>), grid, dim3(kRefreshThreads), lds, st, d_chunks, so); break;
        case ELX_BF16: hipLaunchKernelGGL((refresh_kernel<ELX_BF16>), grid, dim3(kRefreshThreads), lds, st, d_chunks, so); break;
        default: return ELX_E_DTYPE;
    }
    return (int)hipGetLastError();
}

uint32_t elx_refresh_piece_elems(void) { return kRefreshPiece; }

int elx_writeback(const float *master, void *lowp, int lowp_dtype, uint64_t n, void *stream) {
    if (!master || !lowp) return ELX_E_NULL;
    if (!is_lowp_or_f32(lowp_dtype)) return ELX_E_DTYPE;
    if (n == 0) return ELX_E_SIZE;
    if (((uintptr_t)master & 3u) || ((uintptr_t)lowp & (elem_size(lowp_dtype) - 1))) return ELX_E_ALIGN;
    ElxChunk c = {};
    c.lowp_out = lowp;
    c.master = const_cast<float *>(master);
    c.n_alloc = n;
    const uint32_t so = (((uintptr_t)master | (uintptr_t)lowp) & 15u) ? 1u : 0u;
    const uint64_t pieces = (n + kRefreshPiece - 1) / kRefreshPiece;
    const dim3 grid((uint32_t)(pieces < kMaxRefreshBlocks ? pieces : kMaxRefreshBlocks));
    hipStream_t st = (hipStream_t)stream;
    uint32_t lds = 0;
    if (int rc = occupancy_reservation(kRefreshBlocksPerCu, &lds)) return rc;
    switch (lowp_dtype) {
        case ELX_F32: hipLaunchKernelGGL((refresh_one_kernel<ELX_F32>), grid, dim3(kRefreshThreads), lds, st, c, so); break;
        case ELX_F16: hipLaunchKernelGGL((refresh_one_kernel<ELX_F16>), grid, dim3(kRefreshThreads), lds, st, c, so); break;
        default: hipLaunchKernelGGL((refresh_one_kernel<ELX_BF16>), grid, dim3(kRefreshThreads), lds, st, c, so); break;
    }
    return (int)hipGetLastError();
}

int elx_grad_stats(const void *grad, int grad_dtype, uint64_t n, uint32_t blocks, ElxStats *d_partials,
                   ElxStats *d_stats, void *stream) {
    if (!d_partials || !d_stats || (!grad && n)) return ELX_E_NULL;
    if (!is_lowp_or_f32(grad_dtype)) return ELX_E_DTYPE;
    if (blocks == 0 || blocks > kMaxStatsBlocks) return ELX_E_SIZE;
    if ((uintptr_t)grad & (elem_size(grad_dtype) - 1)) return ELX_E_ALIGN;
    ElxChunk c = {};
    c.grad = grad;
    c.n_alloc = n;
    c.n_valid = n;
    const uint32_t so = ((uintptr_t)grad & 15u) ? 1u : 0u;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid(blocks);
    switch (grad_dtype) {
        case ELX_F32: hipLaunchKernelGGL((grad_stats_one_kernel<ELX_F32>), grid, dim3(kStatsThreads), 0, st, c, blocks, d_partials, so); break;
        case ELX_F16: hipLaunchKernelGGL((grad_stats_one_kernel<ELX_F16>), grid, dim3(kStatsThreads), 0, st, c, blocks, d_partials, so); break;
        default: hipLaunchKernelGGL((grad_stats_one_kernel<ELX_BF16>), grid, dim3(kStatsThreads), 0, st, c, blocks, d_partials, so); break;
    }
    int rc = (int)hipGetLastError();
    if (rc) return rc;
    hipLaunchKernelGGL(stats_finish_kernel, dim3(1), dim3(kStatsThreads), 0, st, d_partials, blocks, d_stats);
    return (int)hipGetLastError();
}

int elx_land_grads_mt(const ElxChunk *d_rows, uint32_t n_rows, const uint32_t *d_slot_offsets, uint32_t n_slots,
                      int src_dtype, int dst_dtype, float mul, uint32_t blocks_per_row, ElxStats *d_partials,
                      ElxStats *d_stats, uint32_t flags, void *stream) {
    if (!d_rows || !d_partials || !d_stats) return ELX_E_NULL;
    if (!is_lowp_or_f32(src_dtype) || !is_lowp_or_f32(dst_dtype)) return ELX_E_DTYPE;
    if (src_dtype != dst_dtype && src_dtype != ELX_F32) return ELX_E_DTYPE;
    if (n_rows == 0 || n_rows > 65535u || blocks_per_row == 0 || blocks_per_row > kMaxLandBlocks) return ELX_E_SIZE;
    if (!d_slot_offsets) n_slots = n_rows;
    if (n_slots == 0 || n_slots > n_rows) return ELX_E_SIZE;
    if (!(mul == mul) || mul <= 0.0f || mul > 3.0e38f) return ELX_E_RANGE;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const dim3 grid(blocks_per_row, n_rows);
    const uint32_t so = (flags & ELX_FLAG_SCALAR_ONLY) ? 1u : 0u;
    uint32_t lds = 0;
    const uint32_t land_default = (src_dtype == ELX_F32 && dst_dtype != ELX_F32) ? kDefaultLandBlocksPerCuNarrowing
                                                                                 : kDefaultLandBlocksPerCu;
    int rc = occupancy_reservation(((flags >> 8) & 0xFFu) ? ((flags >> 8) & 0xFFu) : land_default, &lds);
    if (rc) return rc;
    rc = ELX_E_DTYPE;
#define ELX_LAND(S, D)                                                                                       \
    if (src_dtype == S && dst_dtype == D)                                                                    \
        rc = launch_land<S, D>(mul != 1.0f, (flags & ELX_FLAG_KEEP_CACHED) != 0, grid, lds, st, d_rows, mul,    \
                               d_partials, so);
    ELX_LAND(ELX_F32, ELX_F32)
    ELX_LAND(ELX_F16, ELX_F16)
    ELX_LAND(ELX_BF16, ELX_BF16)
    ELX_LAND(ELX_F32, ELX_F16)
    ELX_LAND(ELX_F32, ELX_BF16)
#undef ELX_LAND
    if (rc) return rc;
    // one slot per row and few partials: the finish alone; otherwise two stages
    if (!d_slot_offsets && blocks_per_row <= kFoldThreshold) {
        hipLaunchKernelGGL(stats_finish_kernel, dim3(n_rows), dim3(kStatsThreads), 0, st, d_partials, blocks_per_row, d_stats);
        return (int)hipGetLastError();
    }
    ElxStats *mid = d_partials + (uint64_t)n_rows * blocks_per_row;
    hipLaunchKernelGGL(stats_fold_kernel, dim3(kFoldBlocks, n_slots), dim3(kStatsThreads), 0, st, d_partials,
                       blocks_per_row, d_slot_offsets, mid);
    rc = (int)hipGetLastError();
    if (rc) return rc;
    hipLaunchKernelGGL(stats_finish_kernel, dim3(n_slots), dim3(kStatsThreads), 0, st, mid, kFoldBlocks, d_stats);
    return (int)hipGetLastError();
}

uint32_t elx_land_fold_blocks(void) { return kFoldBlocks; }

}    // extern "C"
