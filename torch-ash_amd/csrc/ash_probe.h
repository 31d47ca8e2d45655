// Read side of the table for kernels outside ash_map.hip as well: slot
// addressing, the look-up in the second region, and the look-up of one key by
// one lane on its own.
#pragma once

#include "ash_table.h"

namespace ash {

__device__ __forceinline__ unsigned long long* slot_ptr(const MapDev& m,
                                                        uint32_t b, int s) {
    return reinterpret_cast<unsigned long long*>(
            m.buckets + static_cast<size_t>(b) * kBucketQwords + s);
}

__device__ __forceinline__ int32_t* value_ptr(const MapDev& m, uint32_t b,
                                              int s) {
    return reinterpret_cast<int32_t*>(m.buckets) +
           static_cast<size_t>(b) * kBucketDwords + kValDword0 + s;
}

// ------------------------------------------- general (exotic) region, reads
template <int DIM>
__device__ __forceinline__ uint32_t gen_home(const int32_t (&k)[DIM],
                                             uint32_t gslots) {
    uint64_t h = 0xcbf29ce484222325ull;
#pragma unroll
    for (int d = 0; d < DIM; ++d) {
        h ^= static_cast<uint32_t>(k[d]);
        h *= 0x100000001b3ull;
    }
    return static_cast<uint32_t>(mix64(h)) & (gslots - 1);
}

__device__ __forceinline__ int32_t gen_load(const int32_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int DIM>
__device__ __forceinline__ bool gen_key_equal(const MapDev& m, uint32_t p,
                                              const int32_t (&k)[DIM]) {
    bool eq = true;
#pragma unroll
    for (int d = 0; d < DIM; ++d) {
        eq = eq && (gen_load(m.gkeys + static_cast<size_t>(p) * 4 + d) == k[d]);
    }
    return eq;
}

// Returns true and the stored index when the key is present.
template <int DIM>
__device__ bool gen_find(const MapDev& m, const int32_t (&k)[DIM],
                         int32_t& idx, uint32_t& pos) {
    if (m.gstate == nullptr) return false;
    const uint32_t mask = m.gslots - 1;
    uint32_t p = gen_home<DIM>(k, m.gslots);
    for (uint32_t step = 0; step < m.gslots; ++step) {
        const int32_t w = gen_load(m.gstate + p);
        if (w == kGenEmpty) return false;
        if (w >= 0 && gen_key_equal<DIM>(m, p, k)) {
            idx = w;
            pos = p;
            return true;
        }
        p = (p + 1) & mask;
    }
    return false;
}

// Look-up of one key by one lane on its own (the cooperative probe of
// ash_map.hip shares a bucket read among eight lanes): the lane reads the ten
// codes of the key's bucket itself (five 16-byte loads of one 128-byte line).  Far fewer vector
// instructions per wavefront than the cooperative probe, at the price of one
// line per lane and load instruction; for kernels whose table is small enough
// to stay in the caches and that are bound by instructions, not by lines.
template <int DIM>
__device__ __forceinline__ bool find_key_alone(const MapDev& m, const int32_t (&k)[DIM],
                                               bool active, int32_t& res) {
    static_assert(kSlots == 10, "reads the codes as five 16-byte words");
    uint64_t code;
    const bool fits = pack_key<DIM>(k, code);
    bool pend = active && fits;
    uint32_t b = bucket_of(code, m.nb);
    uint32_t steps = 0;
    res = 0;
    bool found = false;
    while (pend) {
        const uint4* line = reinterpret_cast<const uint4*>(
                m.buckets + static_cast<size_t>(b) * kBucketQwords);
        uint4 w[5];
#pragma unroll
        for (int r = 0; r < 5; ++r) w[r] = line[r];
        int slot = -1;
        bool empty = false;
#pragma unroll
        for (int r = 4; r >= 0; --r) {
            const uint64_t qa = static_cast<uint64_t>(w[r].x) | (static_cast<uint64_t>(w[r].y) << 32);
            const uint64_t qb = static_cast<uint64_t>(w[r].z) | (static_cast<uint64_t>(w[r].w) << 32);
            empty = empty || qa == kEmpty || qb == kEmpty;
            if (qb == code) slot = 2 * r + 1;
            if (qa == code) slot = 2 * r;
        }
        if (slot >= 0) {
            found = true;
            res = *value_ptr(m, b, slot);
            pend = false;
        } else if (empty) {
            pend = false;
        } else {
            b = next_bucket(b, m.nb);
            if (++steps >= kPartBuckets) pend = false;
        }
    }
    if (active && !fits) {
        uint32_t pos;
        found = gen_find<DIM>(m, k, res, pos);
    }
    return found;
}

// A position x (cell units, fp32) split into block / cell / fractional part as
// SparseDenseGrid.query does (ash/grid.py:183-199), one axis.  The arithmetic
// is the reference's torch expression evaluated operation by operation in fp32
// (no fused multiply-add, so the results equal the elementwise torch
// formulation bit for bit):
//   xs = floor(x / G); xd = x - xs * G; off = xd - floor(xd)
// with two corrections at block boundaries, where fp32 rounding takes xd out
// of [0, G): xd < 0 (x / G rounded up to an integer) steps back one block,
// xd == G (tiny negative x) is cell 0 of the next block.
__device__ __forceinline__ void split_axis(float xv, float g, int32_t& block, int32_t& cell,
                                           float& off) {
    float xs = floorf(__fdiv_rn(xv, g));
    float xd = __fsub_rn(xv, __fmul_rn(xs, g));
    const float under = xd < 0.f ? 1.f : 0.f;
    xs = __fsub_rn(xs, under);
    xd = __fadd_rn(xd, __fmul_rn(under, g));
    const float spill = xd >= g ? 1.f : 0.f;
    xs = __fadd_rn(xs, spill);
    xd = __fsub_rn(xd, __fmul_rn(spill, g));
    off = __fsub_rn(xd, floorf(xd));
    block = static_cast<int32_t>(xs);
    cell = static_cast<int32_t>(xd);
}

// Look-up of the blocks of 64 positions held by a wavefront, one per lane.
// Neighbouring positions (samples along a ray) often stand in the same block:
// the first lane of a run of equal keys looks the block up, by itself, and the
// others take its answer.  Every lane of the wavefront must take part.
__device__ __forceinline__ bool find_block_by_runs(const MapDev& m, const int32_t (&k)[3],
                                                   bool active, int32_t& res) {
    const int lane = threadIdx.x & 63;
    int same = lane > 0;
#pragma unroll
    for (int d = 0; d < 3; ++d) same &= __shfl_up(k[d], 1) == k[d];
    const bool head = !same;
    const bool asked = find_key_alone<3>(m, k, active && head, res);
    const uint64_t heads = __ballot(head);
    const int my_head = 63 - __builtin_clzll(heads & (~0ull >> (63 - lane)));
    const bool found = __shfl(static_cast<int>(asked), my_head) != 0;
    res = __shfl(res, my_head);
    return found;
}

}  // namespace ash
