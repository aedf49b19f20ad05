// The parts of the library that run on the host and need no GPU runtime: the constants that fix the
// shape of the launches, how a launch divides by div_scale, the LDS reservation that caps residency,
// and the validators that stand between a caller's tables and a launch.  elx_host.cpp holds the
// code; it is linked into libelx_hip.so and also compiles on its own with a plain C++ compiler, which
// is how the validators are run under AddressSanitizer / UBSan.
#ifndef ELX_HOST_H
#define ELX_HOST_H

#include <stdint.h>

#include "elx_abi.h"

namespace elx_host {

constexpr int kWave = 64;                              // one wavefront per update workgroup
constexpr int kVec = 4;                                // elements per lane per access
constexpr int kUnroll = 1;                             // independent accesses per lane per stream
constexpr uint32_t kSpan = kWave * kVec;               // elements one wavefront access covers
constexpr uint32_t kTile = kSpan * kUnroll;            // 256 elements per tile
constexpr uint64_t kMaxBufferElems = 1ull << 40;       // longest buffer a table row may describe (tile arithmetic stays far from overflow)
constexpr uint32_t kLdsPerCu = 160u * 1024u;           // gfx950
constexpr uint32_t kDefaultBlocksPerCu = 12;           // fp32 gradients (4 KiB of loads in flight per workgroup)
constexpr uint32_t kDefaultBlocksPerCuLowp = 13;       // 16-bit gradients (3.5 KiB): one more workgroup pays
constexpr uint32_t kMinBlocksPerCu = 3;                // keeps the reservation below 64 KiB
constexpr uint32_t kMaxBlocksPerCu = 32;

constexpr int kLandUnroll = 4;                         // 128-bit loads per lane of one landing tile
constexpr uint32_t kMaxLandBlocks = 1u << 20;

// How the gradient is unscaled: not at all, by an exact multiply with 1/div_scale (div_scale a
// power of two: same bits as the division), or by a true IEEE division.
enum { kDivNone = 0, kDivMulInv = 1, kDivTrue = 2 };

struct Unscale {
    float div_scale, inv_scale;
    int mode;
};

bool is_lowp_or_f32(int d);
uint32_t elem_size(int d);

// div_scale is a power of two whose reciprocal is a normal fp32 number
bool exact_reciprocal(float s);

// How the update launch divides by div_scale (the div_scale of optimizer.py:216; <= 0: not at all).
Unscale unscale_of(float div_scale);

// dynamic LDS bytes that let exactly `blocks_per_cu` update workgroups share a compute unit
int occupancy_reservation(uint32_t blocks_per_cu, uint32_t *lds_bytes, uint32_t fallback = kDefaultBlocksPerCu);

}    // namespace elx_host

#endif    // ELX_HOST_H
