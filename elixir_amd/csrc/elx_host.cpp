// Host-only code of libelx_hip.so (see elx_host.h): no GPU runtime call, no device code.
#include "elx_host.h"

#include <string.h>

namespace elx_host {

bool is_lowp_or_f32(int d) { return d == ELX_F32 || d == ELX_F16 || d == ELX_BF16; }

uint32_t elem_size(int d) { return d == ELX_F32 ? 4u : 2u; }

bool exact_reciprocal(float s) {
    uint32_t u;
    memcpy(&u, &s, 4);
    const uint32_t exp = (u >> 23) & 0xFFu, man = u & 0x7FFFFFu;
    return (u >> 31) == 0 && man == 0 && exp >= 1 && exp <= 252;
}

Unscale unscale_of(float div_scale) {
    Unscale us;
    us.div_scale = div_scale;
    us.inv_scale = 1.0f;
    us.mode = kDivNone;
    if (div_scale > 0.0f) {
        if (exact_reciprocal(div_scale)) {
            us.mode = kDivMulInv;
            us.inv_scale = 1.0f / div_scale;
        } else {
            us.mode = kDivTrue;
        }
    }
    return us;
}

int occupancy_reservation(uint32_t blocks_per_cu, uint32_t *lds_bytes, uint32_t fallback) {
    if (blocks_per_cu == 0) blocks_per_cu = fallback;
    if (blocks_per_cu < kMinBlocksPerCu || blocks_per_cu > kMaxBlocksPerCu) return ELX_E_SIZE;
    *lds_bytes = (kLdsPerCu / blocks_per_cu) & ~255u;
    return 0;
}

}    // namespace elx_host

using namespace elx_host;

extern "C" {

int elx_check_tables(const ElxChunk *h_chunks, uint32_t n_chunks, const ElxSeg *h_segs, uint32_t n_segs,
                     uint32_t n_hypers, int grad_dtype, int lowp_dtype, uint64_t *total_tiles,
                     uint32_t *max_tiles_per_chunk, int *all_aligned16) {
    if (!h_chunks || !total_tiles || !max_tiles_per_chunk || !all_aligned16 || (n_segs && !h_segs)) return ELX_E_NULL;
    if (n_chunks == 0 || n_chunks > 65535u) return ELX_E_SIZE;
    if (!is_lowp_or_f32(grad_dtype)) return ELX_E_DTYPE;
    if (lowp_dtype != ELX_NONE && lowp_dtype != grad_dtype) return ELX_E_DTYPE;
    const uintptr_t gmask = elem_size(grad_dtype) - 1;
    uint64_t tiles = 0;
    int aligned = 1;
    uint64_t max_tiles = 0;
    for (uint32_t i = 0; i < n_chunks; ++i) {
        const ElxChunk &c = h_chunks[i];
        if (!c.master || !c.m || !c.v) return ELX_E_NULL;
        if (c.lowp_out && lowp_dtype == ELX_NONE) return ELX_E_DTYPE;
        if (c.n_alloc == 0 || c.n_alloc > kMaxBufferElems) return ELX_E_SIZE;
        if ((c.n_alloc + kTile - 1) / kTile > max_tiles) max_tiles = (c.n_alloc + kTile - 1) / kTile;
        if (c.n_valid > c.n_alloc) return ELX_E_RANGE;
        const uintptr_t ptrs[5] = {(uintptr_t)c.grad, (uintptr_t)c.lowp_out, (uintptr_t)c.master, (uintptr_t)c.m,
                                   (uintptr_t)c.v};
        if ((ptrs[0] & gmask) || (ptrs[1] & gmask) || (ptrs[2] & 3u) || (ptrs[3] & 3u) || (ptrs[4] & 3u))
            return ELX_E_ALIGN;
        for (int k = 0; k < 5; ++k)
            if (ptrs[k] & 15u) aligned = 0;
        if (c.tile_begin != tiles) return ELX_E_TILES;
        tiles += (c.n_alloc + kTile - 1) / kTile;
        if (c.seg_begin > c.seg_end || c.seg_end > n_segs) return ELX_E_RANGE;
        uint64_t prev_end = 0;
        for (uint32_t s = c.seg_begin; s < c.seg_end; ++s) {
            const ElxSeg &sg = h_segs[s];
            if (sg.begin >= sg.end || sg.end > c.n_valid) return ELX_E_RANGE;
            if (sg.hyper >= n_hypers) return ELX_E_RANGE;
            if (sg.begin < prev_end) return ELX_E_ORDER;
            prev_end = sg.end;
        }
    }
    if (tiles > 0x7FFFFFFFull) return ELX_E_SIZE;    // one workgroup per tile
    *total_tiles = tiles;
    *max_tiles_per_chunk = (uint32_t)max_tiles;
    *all_aligned16 = aligned;
    return 0;
}

int elx_check_land_rows(const ElxChunk *h_rows, uint32_t n_rows, const uint32_t *h_slot_offsets, uint32_t n_slots,
                        int src_dtype, int dst_dtype, uint32_t *blocks_per_row) {
    if (!h_rows || !blocks_per_row) return ELX_E_NULL;
    if (!is_lowp_or_f32(src_dtype) || !is_lowp_or_f32(dst_dtype)) return ELX_E_DTYPE;
    if (src_dtype != dst_dtype && src_dtype != ELX_F32) return ELX_E_DTYPE;
    if (n_rows == 0 || n_rows > 65535u) return ELX_E_SIZE;
    const uintptr_t smask = elem_size(src_dtype) - 1, dmask = elem_size(dst_dtype) - 1;
    const uint64_t tile = kWave * (16u / elem_size(src_dtype)) * kLandUnroll;
    uint64_t max_tiles = 1;
    for (uint32_t i = 0; i < n_rows; ++i) {
        const ElxChunk &r = h_rows[i];
        if (!r.lowp_out) return ELX_E_NULL;
        if (r.n_alloc == 0 || r.n_alloc > kMaxBufferElems) return ELX_E_SIZE;
        if (r.n_valid > r.n_alloc) return ELX_E_RANGE;
        if (((uintptr_t)r.grad & smask) || ((uintptr_t)r.lowp_out & dmask)) return ELX_E_ALIGN;
        const uint64_t t = (r.n_alloc + tile - 1) / tile;
        if (t > max_tiles) max_tiles = t;
    }
    if (h_slot_offsets) {
        if (n_slots == 0 || n_slots > n_rows) return ELX_E_SIZE;
        if (h_slot_offsets[0] != 0 || h_slot_offsets[n_slots] != n_rows) return ELX_E_RANGE;
        for (uint32_t s = 0; s < n_slots; ++s)
            if (h_slot_offsets[s] > h_slot_offsets[s + 1]) return ELX_E_ORDER;
    }
    // a row with more tiles than a launch may have workgroups per row: each workgroup takes several
    *blocks_per_row = (uint32_t)(max_tiles < kMaxLandBlocks ? max_tiles : kMaxLandBlocks);
    return 0;
}

int elx_unscale_mode(float div_scale, float *inv_scale) {
    const Unscale us = unscale_of(div_scale);
    if (inv_scale) *inv_scale = us.inv_scale;
    return us.mode;
}

int elx_occupancy_lds_bytes(uint32_t blocks_per_cu, uint32_t *lds_bytes) {
    if (!lds_bytes) return ELX_E_NULL;
    return occupancy_reservation(blocks_per_cu, lds_bytes);
}

uint32_t elx_tile_elems(void) { return kTile; }

uint32_t elx_land_tile_elems(int src_dtype) { return kWave * (16u / elem_size(src_dtype)) * kLandUnroll; }

uint32_t elx_land_max_blocks(void) { return kMaxLandBlocks; }

const char *elx_source_sha(void) {
#ifdef ELX_SOURCE_SHA
    return ELX_SOURCE_SHA;
#else
    return "";
#endif
}

}    // extern "C"
