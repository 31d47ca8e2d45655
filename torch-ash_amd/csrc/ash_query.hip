// Trilinear query kernels of libash_hip.so (gfx950): forward, backward and
// double backward of the sparse-dense grid interpolation
//   y[i,:] = sum_c w_c(offset_i) * embeddings[g_c, cell_c, :]
// with the reference's addressing (ash/src/grid.cu:68-132): the 8 corner rows
// of query i are found through three neighbour tables,
//   nbn = lut_cell_nb2grid_nb[cell_i][c]     which neighbour block (0..7)
//   g_c = lut_grid_nb2grid_idx[grid_i][nbn]  its block index, -1 if missing
//   cell_c = lut_cell_nb2cell_idx[cell_i][c] the cell inside that block
// and a query with any missing neighbour block yields zeros.
//
// Structure.  A workgroup of 256 threads takes tiles of 256 queries.
//   Phase 1 (one thread per query) reads the query's indices, offsets and mask
//   with coalesced loads, walks the neighbour tables (the two per-cell tables
//   are staged once per workgroup in LDS as uint16/uint8) and leaves the 8 row
//   numbers g_c * M + cell_c and the 3 offsets of every query in LDS.
//   Phase 2 re-maps the threads so that LPQ lanes share one query and each lane
//   owns VEC consecutive channels: one request of a wavefront then covers whole
//   embedding rows (E = 16 fp32: 4 lanes x 16 B = one 64-byte row, 16 rows per
//   instruction, 1 KiB of contiguous output), and the per-query address work is
//   not repeated per channel.  When one lane covers the row (LPQ = 1) both
//   phases run in registers without the LDS round trip.
// Workgroups are persistent and walk the tiles of "their" XCD (workgroup id
// mod 8), so neighbouring queries meet in one L2.  Gradients for the embeddings
// are accumulated with hardware floating-point atomics; consecutive queries of
// a wavefront that hit the same row are summed in registers first and issue
// one atomic per run (ray-ordered samples produce long runs).
#include "ash_probe.h"

#include <type_traits>

#include <hip/amd_detail/amd_hip_unsafe_atomics.h>

#include <cmath>
#include <cstdlib>

#include "../../include/ash_hip.h"

namespace ash {
namespace {

constexpr int kBlock = 256;
constexpr int kXcds = 8;
constexpr int64_t kMaxLdsCells = 2048;  // 2048 * 8 * 3 B = 48 KiB
constexpr uint32_t kNoRow = 0xFFFFFFFFu;
constexpr int kLdsPerCu = 160 * 1024;
// Wavefronts per SIMD the kernels are compiled for: the highest occupancy that
// needs no register spills (measured: spilling costs more than the extra
// wavefronts bring).  The one-lane-per-query gather fits 4, the
// channel-parallel kernels, which hold 8 rows plus the run-merge state per
// lane, fit 3.
constexpr int kWavesGather = 4;
constexpr int kWavesWide = 3;

struct QDev {
    const void* emb;
    const float* off;
    const int64_t* gidx;
    const int64_t* cidx;
    const uint8_t* mask;
    const int64_t* lut_g;
    const int64_t* lut_c2c;
    const int64_t* lut_c2g;
    int64_t N;
    int64_t B;
    int64_t M;
    int E;
    int smooth;    // 0 linear, 1 smooth step
    int merge;     // pre-reduce runs of equal rows before the atomics
};

// Interpolation basis (ash/src/grid.cu:7-41).
template <typename T>
__device__ __forceinline__ T basis(T x, int smooth) {
    return smooth ? x * x * (T(3) - T(2) * x) : x;
}
template <typename T>
__device__ __forceinline__ T dbasis(T x, int smooth) {
    return smooth ? T(6) * x * (T(1) - x) : T(1);
}

// Per-axis factors of the corner weights and of their derivatives
// (ash/src/grid.cu:113-118,229-241): side 0 is the "1 - o" side.
template <typename T>
struct AxisTerms {
    T w[3][2];
    T dw[3][2];
};

template <typename T, bool GRAD>
__device__ __forceinline__ void axis_terms(const float (&o)[3], int smooth,
                                           AxisTerms<T>& t) {
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        const T x1 = static_cast<T>(o[d]);
        const T x0 = static_cast<T>(1.0f - o[d]);
        t.w[d][0] = basis<T>(x0, smooth);
        t.w[d][1] = basis<T>(x1, smooth);
        if constexpr (GRAD) {
            t.dw[d][0] = -dbasis<T>(x0, smooth);
            t.dw[d][1] = dbasis<T>(x1, smooth);
        }
    }
}

template <typename T>
__device__ __forceinline__ T corner_weight(const AxisTerms<T>& t, int c) {
    T w = T(1);
    w *= t.w[0][c & 1];
    w *= t.w[1][(c >> 1) & 1];
    w *= t.w[2][(c >> 2) & 1];
    return w;
}

template <typename T>
__device__ __forceinline__ void corner_weight_grad(const AxisTerms<T>& t, int c,
                                                   T (&g)[3]) {
    const int b0 = c & 1, b1 = (c >> 1) & 1, b2 = (c >> 2) & 1;
    g[0] = t.dw[0][b0] * t.w[1][b1] * t.w[2][b2];
    g[1] = t.w[0][b0] * t.dw[1][b1] * t.w[2][b2];
    g[2] = t.w[0][b0] * t.w[1][b1] * t.dw[2][b2];
}

// ------------------------------------------------------------ LDS layout
// [ tile: row[8][256] uint32, off[3][256] float ]  (only when LPQ > 1)
// [ per-cell tables: c2c[M*8] uint16, c2g[M*8] uint8 ]  (only when lds_lut)
// [ one LineTable per wavefront ]  (E = 4 backward kernels that produce grad_embeddings)
struct Tile {
    uint32_t row[8][kBlock];
    float off[3][kBlock];
};

struct CellLut {
    const uint16_t* c2c;
    const uint8_t* c2g;
};

template <bool LDS>
__device__ __forceinline__ void cell_neighbor(const QDev& a, const CellLut& lut,
                                              int64_t cell, int c, int& nb_cell,
                                              int& nb_grid) {
    if constexpr (LDS) {
        nb_cell = lut.c2c[cell * 8 + c];
        nb_grid = lut.c2g[cell * 8 + c];
    } else {
        int64_t v = a.lut_c2c[cell * 8 + c];
        v = v < 0 ? 0 : (v >= a.M ? a.M - 1 : v);
        nb_cell = static_cast<int>(v);
        nb_grid = static_cast<int>(a.lut_c2g[cell * 8 + c]) & 7;
    }
}

template <bool LDS>
__device__ __forceinline__ CellLut stage_cell_lut(const QDev& a,
                                                  unsigned char* smem) {
    CellLut lut;
    lut.c2c = nullptr;
    lut.c2g = nullptr;
    if constexpr (LDS) {
        uint16_t* s_c2c = reinterpret_cast<uint16_t*>(smem);
        uint8_t* s_c2g = smem + a.M * 8 * 2;
        const int64_t n = a.M * 8;
        for (int64_t t = threadIdx.x; t < n; t += kBlock) {
            int64_t v = a.lut_c2c[t];
            v = v < 0 ? 0 : (v >= a.M ? a.M - 1 : v);
            s_c2c[t] = static_cast<uint16_t>(v);
            s_c2g[t] = static_cast<uint8_t>(a.lut_c2g[t] & 7);
        }
        __syncthreads();
        lut.c2c = s_c2c;
        lut.c2g = s_c2g;
    }
    return lut;
}

// Where the line tables of the float4 backward kernels start in dynamic LDS.
__host__ __device__ inline size_t table_offset(const QDev& a, int lpq, bool lds_lut) {
    size_t bytes = lpq > 1 ? sizeof(Tile) : 0;
    if (lds_lut) bytes += static_cast<size_t>(a.M) * 8 * 3;
    return (bytes + 15) & ~static_cast<size_t>(15);
}

// Tile walk: workgroup w serves XCD (w mod 8); each XCD owns a contiguous
// eighth of the tiles and its workgroups stride through it.
struct TileWalk {
    int64_t next;
    int64_t end;
    int64_t step;
    __device__ __forceinline__ TileWalk(int64_t ntiles) {
        const int64_t per_xcd = (ntiles + kXcds - 1) / kXcds;
        const int xcd = blockIdx.x % kXcds;
        const int slot = blockIdx.x / kXcds;
        step = (gridDim.x + kXcds - 1 - xcd) / kXcds;  // workgroups on this XCD
        next = xcd * per_xcd + slot;
        end = (xcd + 1) * per_xcd;
        if (end > ntiles) end = ntiles;
        if (step < 1) step = 1;
    }
};

// What a query brings.  The mask, the indices and the offsets are asked for
// together (one trip to memory, not two); what a masked query has there is read
// and dropped.  They are read once, like z, and the per-query outputs are
// written once: those loads and stores carry the non-temporal hint, which
// leaves the caches to the embedding rows (forward, E = 4: 0.129 -> 0.117 ms).
struct QueryInputs {
    // low dwords of the int64 indices: a row of the block table is below 2^31
    // and "none" is -1, a cell is below 2^31 too
    int32_t gi, ci;
    float o[3];
    uint8_t m;   // 0: masked out or beyond the last query
};

__device__ __forceinline__ QueryInputs load_inputs(const QDev& a, int64_t q) {
    QueryInputs in;
    in.gi = in.ci = 0;
    in.o[0] = in.o[1] = in.o[2] = 0.f;
    in.m = 0;
    if (q < a.N) {
        in.m = __builtin_nontemporal_load(a.mask + q);
        in.gi = __builtin_nontemporal_load(reinterpret_cast<const int32_t*>(a.gidx) + q * 2);
        in.ci = __builtin_nontemporal_load(reinterpret_cast<const int32_t*>(a.cidx) + q * 2);
        in.o[0] = __builtin_nontemporal_load(a.off + q * 3 + 0);
        in.o[1] = __builtin_nontemporal_load(a.off + q * 3 + 1);
        in.o[2] = __builtin_nontemporal_load(a.off + q * 3 + 2);
    }
    return in;
}

// Phase 1 for one query: the 8 corner rows (kNoRow in row[0] when the query is
// masked out, out of range, or misses a neighbour block) and the offsets.
template <bool LDS>
__device__ __forceinline__ void resolve_rows(const QDev& a, const CellLut& lut,
                                             const QueryInputs& in, uint32_t (&row)[8],
                                             float (&o)[3]) {
    bool valid = in.m != 0 && static_cast<uint32_t>(in.gi) < static_cast<uint32_t>(a.B);
    const int64_t gi = valid ? in.gi : 0;
#pragma unroll
    for (int d = 0; d < 3; ++d) o[d] = valid ? in.o[d] : 0.f;
    const int64_t ci = in.ci < 0 ? 0 : (in.ci >= a.M ? a.M - 1 : in.ci);
    // Block indices are below 2^31 and a missing block is -1, so the low
    // dword of each int64 table entry carries everything.
    const int32_t* lut_g32 = reinterpret_cast<const int32_t*>(a.lut_g) + gi * 16;
    int32_t g0 = -1;
    if (valid) g0 = lut_g32[0];
    const uint32_t nblocks = static_cast<uint32_t>(a.B);
    const uint32_t cells = static_cast<uint32_t>(a.M);
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        row[c] = 0;
        if (valid) {
            int nb_cell, nb_grid;
            cell_neighbor<LDS>(a, lut, ci, c, nb_cell, nb_grid);
            int32_t g = g0;
            if (nb_grid != 0) g = lut_g32[nb_grid * 2];
            if (static_cast<uint32_t>(g) >= nblocks) {
                valid = false;
            } else {
                row[c] = static_cast<uint32_t>(g) * cells +
                         static_cast<uint32_t>(nb_cell);
            }
        }
    }
    if (!valid) row[0] = kNoRow;
}

template <bool LDS>
__device__ __forceinline__ void resolve_rows(const QDev& a, const CellLut& lut,
                                             int64_t q, uint32_t (&row)[8],
                                             float (&o)[3]) {
    resolve_rows<LDS>(a, lut, load_inputs(a, q), row, o);
}

// Runs phase 1 for the tile and hands every thread the rows / offsets of the
// query it serves in pass `p` of phase 2.
template <int LPQ, bool LDS>
struct TileStage {
    static constexpr int kPasses = LPQ;

    static __device__ __forceinline__ void fill(const QDev& a,
                                                const CellLut& lut,
                                                int64_t tile, Tile* s,
                                                uint32_t (&row)[8],
                                                float (&o)[3]) {
        fill_from(a, lut, load_inputs(a, tile * kBlock + threadIdx.x), s, row, o);
    }

    // `in`: what the calling thread's query of the tile brings (read from the
    // operand arrays, or worked out from a position by the fused front end)
    static __device__ __forceinline__ void fill_from(const QDev& a,
                                                     const CellLut& lut,
                                                     const QueryInputs& in, Tile* s,
                                                     uint32_t (&row)[8],
                                                     float (&o)[3]) {
        resolve_rows<LDS>(a, lut, in, row, o);
        if constexpr (LPQ > 1) {
            __syncthreads();  // previous tile fully consumed
#pragma unroll
            for (int c = 0; c < 8; ++c) s->row[c][threadIdx.x] = row[c];
#pragma unroll
            for (int d = 0; d < 3; ++d) s->off[d][threadIdx.x] = o[d];
            __syncthreads();
        }
    }

    static __device__ __forceinline__ int64_t fetch(int64_t tile, int p,
                                                    const Tile* s,
                                                    uint32_t (&row)[8],
                                                    float (&o)[3]) {
        if constexpr (LPQ > 1) {
            // a wavefront serves the 64 consecutive queries it resolved itself,
            // 64 / LPQ of them per pass
            const int qi = (threadIdx.x & ~63) + p * (64 / LPQ) + (threadIdx.x & 63) / LPQ;
#pragma unroll
            for (int c = 0; c < 8; ++c) row[c] = s->row[c][qi];
#pragma unroll
            for (int d = 0; d < 3; ++d) o[d] = s->off[d][qi];
            return tile * kBlock + qi;
        } else {
            return tile * kBlock + threadIdx.x;
        }
    }
};

template <typename T, int VEC>
struct VecOf;
template <>
struct VecOf<float, 4> {
    using type = float4;
};
template <>
struct VecOf<float, 1> {
    using type = float;
};
// Rows of two, three or five fp32 channels taken whole by one lane: a row is
// only 4-byte aligned in general (rows of 12 or 20 bytes follow each other), which is
// all a global load of several dwords asks for on this device.
template <int N>
struct alignas(4) FloatRow {
    float v[N];
};
template <>
struct VecOf<float, 2> {
    using type = FloatRow<2>;
};
template <>
struct VecOf<float, 3> {
    using type = FloatRow<3>;
};
template <>
struct VecOf<float, 5> {
    using type = FloatRow<5>;
};
template <>
struct VecOf<double, 1> {
    using type = double;
};

// ------------------------------------------------------------- forward
// Phase 2 of the forward pass for the query the calling thread serves in pass
// p of the tile: gather of the eight corner rows, weighted sum, one store.
template <typename T, int VEC, int LPQ>
__device__ __forceinline__ void forward_rows(const QDev& a, const T* __restrict__ emb,
                                             T* __restrict__ out, int64_t q,
                                             const uint32_t (&row)[8], const float (&o)[3],
                                             int ch0, bool chv) {
    using V = typename VecOf<T, VEC>::type;
    const bool valid = row[0] != kNoRow;
    alignas(16) T acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = T(0);
    if (valid && chv) {
        V e[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            e[c] = *reinterpret_cast<const V*>(
                    emb + static_cast<int64_t>(row[c]) * a.E + ch0);
        }
        AxisTerms<T> t;
        axis_terms<T, false>(o, a.smooth, t);
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const T w = corner_weight<T>(t, c);
            const T* ev = reinterpret_cast<const T*>(&e[c]);
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[v] += w * ev[v];
        }
    }
    if (q < a.N && chv) {
        if constexpr (sizeof(V) == 16) {
            typedef float v4f __attribute__((ext_vector_type(4)));
            const v4f r4 = {static_cast<float>(acc[0]), static_cast<float>(acc[VEC > 1 ? 1 : 0]),
                            static_cast<float>(acc[VEC > 2 ? 2 : 0]), static_cast<float>(acc[VEC > 3 ? 3 : 0])};
            __builtin_nontemporal_store(r4, reinterpret_cast<v4f*>(out + q * a.E + ch0));
        } else {
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                __builtin_nontemporal_store(acc[v], out + q * a.E + ch0 + v);
            }
        }
    }
}

template <typename T, int VEC, int LPQ, bool LDS>
__global__ __launch_bounds__(kBlock, (LPQ == 1 && VEC <= 4) ? kWavesGather : kWavesWide) void
query_forward_kernel(
        QDev a, T* __restrict__ out) {
    extern __shared__ __align__(16) unsigned char smem[];
    Tile* tile_s = reinterpret_cast<Tile*>(smem);
    const CellLut lut =
            stage_cell_lut<LDS>(a, smem + (LPQ > 1 ? sizeof(Tile) : 0));
    using Stage = TileStage<LPQ, LDS>;
    const int ch0 = (threadIdx.x % LPQ) * VEC;
    const bool chv = ch0 < a.E;
    const T* __restrict__ emb = static_cast<const T*>(a.emb);
    const int64_t ntiles = (a.N + kBlock - 1) / kBlock;
    TileWalk walk(ntiles);
    for (int64_t tile = walk.next; tile < walk.end; tile += walk.step) {
        uint32_t row[8];
        float o[3];
        Stage::fill(a, lut, tile, tile_s, row, o);
#pragma unroll 1
        for (int p = 0; p < Stage::kPasses; ++p) {
            const int64_t q = Stage::fetch(tile, p, tile_s, row, o);
            forward_rows<T, VEC, LPQ>(a, emb, out, q, row, o, ch0, chv);
        }
    }
}

// ------------------------------------------------ forward from positions
// The module-level forward (ash/grid.py:201-238: `query`, then the
// interpolation) in one kernel: the front end of ash_grid_query (position ->
// block / cell / fractional part -> look-up of the block, ash_probe.h) stands
// where the forward kernel reads a query's operands, so the four intermediate
// arrays are neither written nor read back on the way to the result -- they are
// written (once) only for a caller that needs them afterwards: the mask always
// (the module returns it), block index, cell index and offsets when a backward
// pass will want them (AUX).
struct FrontDev {
    MapDev m;
    const float* x;      // float32[N, 3]; cell units = (x - origin) * inv_cell
    const float* origin; // float32[3] on the device, or nullptr for none
    float inv_cell;      // 1 / cell size, rounded to fp32 once
    float g;             // cells per block edge
    int gdim;
    uint8_t* mask_out;   // [N]
    int64_t* gidx_out;   // [N]    (AUX)
    int64_t* cidx_out;   // [N]    (AUX)
    float* off_out;      // [N, 3] (AUX)
};

template <bool AUX>
__device__ __forceinline__ QueryInputs front_inputs(const QDev& a, const FrontDev& f, int64_t q) {
    const bool active = q < a.N;
    QueryInputs in;
    int32_t k[3];
    int32_t cell = 0, stride = 1;
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        int32_t c;
        float xv = active ? __builtin_nontemporal_load(f.x + q * 3 + d) : 0.f;
        // world -> cell units the way torch evaluates `(x - origin) / cell_size`
        // on the device: a subtraction, then a multiplication by the fp32
        // reciprocal of the size (both exact no-ops for origin 0 and size 1)
        xv = __fmul_rn(__fsub_rn(xv, f.origin != nullptr ? f.origin[d] : 0.f), f.inv_cell);
        split_axis(xv, f.g, k[d], c, in.o[d]);
        cell += c * stride;
        stride *= f.gdim;
    }
    int32_t res = 0;
    const bool found = find_block_by_runs(f.m, k, active, res);
    in.gi = found ? res : 0;
    in.ci = cell;
    in.m = (active && found) ? 1 : 0;
    if (active) {
        __builtin_nontemporal_store(in.m, f.mask_out + q);
        if constexpr (AUX) {
            __builtin_nontemporal_store(static_cast<int64_t>(in.gi), f.gidx_out + q);
            __builtin_nontemporal_store(static_cast<int64_t>(cell), f.cidx_out + q);
#pragma unroll
            for (int d = 0; d < 3; ++d) __builtin_nontemporal_store(in.o[d], f.off_out + q * 3 + d);
        }
    }
    return in;
}

template <typename T, int VEC, int LPQ, bool LDS, bool AUX>
__global__ __launch_bounds__(kBlock, (LPQ == 1 && VEC <= 4) ? kWavesGather : kWavesWide) void
grid_forward_kernel(QDev a, FrontDev f, T* __restrict__ out) {
    extern __shared__ __align__(16) unsigned char smem[];
    Tile* tile_s = reinterpret_cast<Tile*>(smem);
    const CellLut lut =
            stage_cell_lut<LDS>(a, smem + (LPQ > 1 ? sizeof(Tile) : 0));
    using Stage = TileStage<LPQ, LDS>;
    const int ch0 = (threadIdx.x % LPQ) * VEC;
    const bool chv = ch0 < a.E;
    const T* __restrict__ emb = static_cast<const T*>(a.emb);
    const int64_t ntiles = (a.N + kBlock - 1) / kBlock;
    TileWalk walk(ntiles);
    for (int64_t tile = walk.next; tile < walk.end; tile += walk.step) {
        uint32_t row[8];
        float o[3];
        Stage::fill_from(a, lut, front_inputs<AUX>(a, f, tile * kBlock + threadIdx.x), tile_s,
                         row, o);
#pragma unroll 1
        for (int p = 0; p < Stage::kPasses; ++p) {
            const int64_t q = Stage::fetch(tile, p, tile_s, row, o);
            forward_rows<T, VEC, LPQ>(a, emb, out, q, row, o, ch0, chv);
        }
    }
}

// ------------------------------------------------- run merge for atomics
// Runs of consecutive queries of a wavefront that lie in the same cell.  Two
// queries meet in the same row at a corner only when they lie in the same
// cell, and then at every corner, so the runs are found once per pass, from
// the row of the cell itself, and the sums over them are taken corner by
// corner: one lane exchange per step and corner.  Query groups are LPQ lanes
// wide (one lane per channel); a lane talks to the lanes of its own channel.
template <int LPQ>
struct GroupRuns {
    static constexpr int kGroups = 64 / LPQ;
    static constexpr int kSteps = kGroups > 32 ? 6 : kGroups > 16 ? 5 : kGroups > 8 ? 4
                                  : kGroups > 4 ? 3 : kGroups > 2 ? 2 : 1;
    bool any;            // some group continues the run of the group before it (the same for all lanes)
    bool take[kSteps];   // step k of the segmented sum adds what lies 2^k groups below
    bool tail;           // the last group of its run: holds the total afterwards
};

// `on`: the lane has a query and a channel.  Every lane of the wavefront must
// take part.
template <int LPQ>
__device__ __forceinline__ GroupRuns<LPQ> find_group_runs(uint32_t cell_row, bool on, int lane) {
    using R = GroupRuns<LPQ>;
    R r;
    const int grp = lane / LPQ;
    // lanes that are off get a row number no neighbour shares
    const uint32_t id = on ? cell_row : (kNoRow - static_cast<uint32_t>(grp & 1));
    const uint32_t prev = __shfl_up(id, LPQ);
    const uint32_t next = __shfl_down(id, LPQ);
    const bool head = (grp == 0) || (prev != id) || !on;
    r.tail = (grp == R::kGroups - 1) || (next != id);
    r.any = __ballot(!head) != 0;
    int f = head ? 1 : 0;
#pragma unroll
    for (int k = 0; k < R::kSteps; ++k) {
        const int d = 1 << k;
        const int fu = __shfl_up(f, d * LPQ);
        r.take[k] = grp >= d && !f;
        if (r.take[k]) f |= fu;
    }
    return r;
}

// Adds v to grad_emb[row, ch] for the lanes that are `on`; with `runs` the
// last group of every run adds the run's sum (runs.any false: every lane for
// itself).  Every lane of the wavefront must take part.
template <typename T, int LPQ>
__device__ __forceinline__ void accumulate_row(T* __restrict__ grad_emb,
                                               uint32_t row, int E, int ch,
                                               bool on, T v, const GroupRuns<LPQ>& runs) {
    bool last = true;
    if (runs.any) {   // (the same for all lanes)
#pragma unroll
        for (int k = 0; k < GroupRuns<LPQ>::kSteps; ++k) {
            const T vu = __shfl_up(v, (1 << k) * LPQ);
            if (runs.take[k]) v += vu;
        }
        last = runs.tail;
    }
    if (on && last) {
        unsafeAtomicAdd(grad_emb + static_cast<int64_t>(row) * E + ch, v);
    }
}

// --------------------------------------------------- backward (first order)
// grad_embeddings[row_c, k] += w_c * z[i,k];
// grad_offsets[i,:] = sum_c (emb[row_c,:] . z[i,:]) * grad w_c
// (ash/src/grid.cu:177-255).  One lane per channel.
// OUT: bit 0 = produce grad_embeddings, bit 1 = produce grad_offsets.
template <typename T, int LPQ, bool LDS, int OUT>
__global__ __launch_bounds__(kBlock, kWavesWide) void
query_backward_forward_kernel(
        QDev a, const T* __restrict__ z, T* __restrict__ grad_emb,
        T* __restrict__ grad_off) {
    extern __shared__ __align__(16) unsigned char smem[];
    Tile* tile_s = reinterpret_cast<Tile*>(smem);
    const CellLut lut =
            stage_cell_lut<LDS>(a, smem + (LPQ > 1 ? sizeof(Tile) : 0));
    using Stage = TileStage<LPQ, LDS>;
    const int lane = threadIdx.x & 63;
    const int ch = threadIdx.x % LPQ;
    const bool chv = ch < a.E;
    const T* __restrict__ emb = static_cast<const T*>(a.emb);
    constexpr bool want_emb = (OUT & 1) != 0;
    constexpr bool want_off = (OUT & 2) != 0;
    const int64_t ntiles = (a.N + kBlock - 1) / kBlock;
    TileWalk walk(ntiles);
    for (int64_t tile = walk.next; tile < walk.end; tile += walk.step) {
        uint32_t row[8];
        float o[3];
        Stage::fill(a, lut, tile, tile_s, row, o);
#pragma unroll 1
        for (int p = 0; p < Stage::kPasses; ++p) {
            const int64_t q = Stage::fetch(tile, p, tile_s, row, o);
            const bool valid = row[0] != kNoRow;
            const bool on = valid && chv;
            const T zk = on ? z[q * a.E + ch] : T(0);
            GroupRuns<LPQ> runs;
            runs.any = false;
            if (want_emb && a.merge) runs = find_group_runs<LPQ>(row[0], on, lane);
            T e[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                e[c] = (on && want_off)
                               ? emb[static_cast<int64_t>(row[c]) * a.E + ch]
                               : T(0);
            }
            AxisTerms<T> t;
            axis_terms<T, true>(o, a.smooth, t);
            T go[3] = {T(0), T(0), T(0)};
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                if constexpr (want_emb) {
                    const T w = corner_weight<T>(t, c);
                    accumulate_row<T, LPQ>(grad_emb, row[c], a.E, ch, on, w * zk, runs);
                }
                if constexpr (want_off) {
                    T gw[3];
                    corner_weight_grad<T>(t, c, gw);
                    T dot = e[c] * zk;
#pragma unroll
                    for (int s = 1; s < LPQ; s <<= 1) dot += __shfl_xor(dot, s);
                    go[0] += dot * gw[0];
                    go[1] += dot * gw[1];
                    go[2] += dot * gw[2];
                }
            }
            if (want_off && q < a.N && ch == 0) {
                grad_off[q * 3 + 0] = valid ? go[0] : T(0);
                grad_off[q * 3 + 1] = valid ? go[1] : T(0);
                grad_off[q * 3 + 2] = valid ? go[2] : T(0);
            }
        }
    }
}

// -------------------------------------------------- backward of backward
// d_c = grad w_c . gg_off[i];  grad_embeddings[row_c,k] += d_c * z[i,k];
// grad_z[i,k] = sum_c d_c * emb[row_c,k]   (ash/src/grid.cu:309-387).
// OUT: bit 0 = produce grad_embeddings, bit 1 = produce grad_z.
template <typename T, int LPQ, bool LDS, int OUT>
__global__ __launch_bounds__(kBlock, kWavesWide) void
query_backward_backward_kernel(
        QDev a, const T* __restrict__ gg_off, const T* __restrict__ z,
        T* __restrict__ grad_z, T* __restrict__ grad_emb) {
    extern __shared__ __align__(16) unsigned char smem[];
    Tile* tile_s = reinterpret_cast<Tile*>(smem);
    const CellLut lut =
            stage_cell_lut<LDS>(a, smem + (LPQ > 1 ? sizeof(Tile) : 0));
    using Stage = TileStage<LPQ, LDS>;
    const int lane = threadIdx.x & 63;
    const int ch = threadIdx.x % LPQ;
    const bool chv = ch < a.E;
    const T* __restrict__ emb = static_cast<const T*>(a.emb);
    constexpr bool want_emb = (OUT & 1) != 0;
    constexpr bool want_z = (OUT & 2) != 0;
    const int64_t ntiles = (a.N + kBlock - 1) / kBlock;
    TileWalk walk(ntiles);
    for (int64_t tile = walk.next; tile < walk.end; tile += walk.step) {
        uint32_t row[8];
        float o[3];
        Stage::fill(a, lut, tile, tile_s, row, o);
#pragma unroll 1
        for (int p = 0; p < Stage::kPasses; ++p) {
            const int64_t q = Stage::fetch(tile, p, tile_s, row, o);
            const bool valid = row[0] != kNoRow;
            const bool on = valid && chv;
            const T zk = on ? z[q * a.E + ch] : T(0);
            GroupRuns<LPQ> runs;
            runs.any = false;
            if (want_emb && a.merge) runs = find_group_runs<LPQ>(row[0], on, lane);
            T gg[3] = {T(0), T(0), T(0)};
            if (valid) {
                gg[0] = gg_off[q * 3 + 0];
                gg[1] = gg_off[q * 3 + 1];
                gg[2] = gg_off[q * 3 + 2];
            }
            T e[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                e[c] = (on && want_z)
                               ? emb[static_cast<int64_t>(row[c]) * a.E + ch]
                               : T(0);
            }
            AxisTerms<T> t;
            axis_terms<T, true>(o, a.smooth, t);
            T gz = T(0);
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                T gw[3];
                corner_weight_grad<T>(t, c, gw);
                const T d = gw[0] * gg[0] + gw[1] * gg[1] + gw[2] * gg[2];
                if constexpr (want_emb) {
                    accumulate_row<T, LPQ>(grad_emb, row[c], a.E, ch, on, d * zk, runs);
                }
                gz += d * e[c];
            }
            if (want_z && q < a.N && chv) {
                grad_z[q * a.E + ch] = on ? gz : T(0);
            }
        }
    }
}

// ================================================== float4 backward kernels
// fp32 embeddings of four channels (a signed distance and a colour, say): one
// lane holds a whole query, as in the forward kernel, so that a wavefront
// serves 64 queries per tile: four times the loads in flight and a quarter of
// the per-query arithmetic of the one-lane-per-channel kernels above.
//
// Gradient rows.  The memory side executes atomics at a fixed rate of
// requests, and one request is what one instruction of a wavefront sends to
// one 64-byte line, whether it carries one float or sixteen (measured: 18 G
// requests/s for 4-byte and for 64-byte groups alike).  The eight corners of a
// query and the queries that follow it along a ray meet the same few lines
// over and over -- the x neighbour is the next row, a corner of this sample is
// another corner of the next -- but in different instructions.  So every
// wavefront first adds its contributions into a small table of lines in LDS
// (open addressing on the line number, sixteen floats per entry) and sends the
// table out once per tile, one line per sixteen lanes: a third of the requests
// on ray-ordered samples.  Before that, runs of consecutive queries with the
// same row are summed in registers (lane exchange inside a row of 16 lanes is
// a modifier of an ordinary vector instruction, across rows it would be a trip
// through the LDS pipeline, so a run is cut at the row of lanes; the table
// joins the pieces).  A row whose line finds no place within kLineProbes steps
// goes to memory directly, and a wavefront that sent more rows that way than
// the table has lines (unordered queries share no lines) leaves the table
// aside for the next kLineRest tiles.
template <int CTRL>
__device__ __forceinline__ int dpp_int(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
template <int CTRL, typename T>
__device__ __forceinline__ T dpp(T v) {
    static_assert(sizeof(T) == 4, "32-bit values");
    return __builtin_bit_cast(T, dpp_int<CTRL>(__builtin_bit_cast(int, v)));
}
constexpr int kRowShl = 0x100;  // lane i takes lane i + n of its row of 16 (0 beyond it)
constexpr int kRowShr = 0x110;  // lane i takes lane i - n

constexpr int kRowBcast15 = 0x142;  // every lane of a row takes lane 15 of the row before

// Runs of consecutive lanes whose queries lie in the same cell.  Two queries
// meet in the same row at a corner only when they lie in the same cell, and
// then at every corner, so the runs are found once per tile, from the row of the
// cell itself, and the sums over them are taken corner by corner (sum_runs).
// The sums run inside the rows of 16 lanes; a run that goes on in the next row
// hands its part over: lane 15 keeps quiet and the lane that ends the run in
// the next row adds what lane 15 had.  (A run that fills a whole row and still
// goes on is not handed over a second time; its parts meet in the table of
// lines.)
struct Runs {
    bool any;         // some lane continues the run of the lane before it (the same for all lanes)
    bool take[4];     // step 1, 2, 4, 8 of the segmented sum adds what lies that far below
    bool takes_offer; // adds what lane 15 of the row before holds
    bool tail;        // this lane ends its run and holds the total
};

// `id`: the row of the query's cell, or for a lane without a query a number no
// neighbour shares.  Every lane of the wavefront must take part.
__device__ __forceinline__ Runs find_runs(uint32_t id, int lane) {
    Runs r;
    const int g = lane & 15;
    const uint32_t prev = dpp<kRowShr + 1>(id);
    const uint32_t next = dpp<kRowShl + 1>(id);
    const bool joins = g > 0 && prev == id;
    r.any = __ballot(joins) != 0;
    const bool starts = g > 0 && prev != id;   // a run starts here, inside the row
    int f = (g == 0 || starts) ? 1 : 0;        // a run starts at or below this lane, as far as summed
    {
        const int fu = dpp_int<kRowShr + 1>(f);
        r.take[0] = g >= 1 && !f;
        if (r.take[0]) f |= fu;
    }
    {
        const int fu = dpp_int<kRowShr + 2>(f);
        r.take[1] = g >= 2 && !f;
        if (r.take[1]) f |= fu;
    }
    {
        const int fu = dpp_int<kRowShr + 4>(f);
        r.take[2] = g >= 4 && !f;
        if (r.take[2]) f |= fu;
    }
    r.take[3] = g >= 8 && !f;
    bool tail = g == 15 || next != id;
    // in the first run of its row: no run starts between the row's first lane and here
    const uint64_t started = __ballot(starts);
    const uint64_t upto = (2ull << lane) - 1ull;
    const uint64_t row_lanes = 0xFFFFull << (lane & 48);
    const bool first_run = (started & upto & row_lanes) == 0;
    // lane 15 offers its sum unless its run began with the row
    const int offers = (g == 15 && !first_run) ? 1 : 0;
    const int offered = dpp_int<kRowBcast15>(offers);
    const uint32_t offered_id = dpp<kRowBcast15>(id);
    r.takes_offer = lane >= 16 && tail && first_run && offered != 0 && offered_id == id;
    // ... and keeps quiet when the next row takes the offer
    const uint32_t id16 = __builtin_amdgcn_readlane(id, 16);
    const uint32_t id32 = __builtin_amdgcn_readlane(id, 32);
    const uint32_t id48 = __builtin_amdgcn_readlane(id, 48);
    const uint32_t over = lane < 16 ? id16 : lane < 32 ? id32 : id48;
    if (offers != 0 && lane < 48 && over == id) tail = false;
    r.tail = tail;
    return r;
}

template <int D>
__device__ __forceinline__ void run_step(float (&v)[4], bool take) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float vu = dpp<kRowShr + D>(v[k]);
        if (take) v[k] += vu;
    }
}

// Sums `v` over the runs; the lanes with r.tail hold the totals afterwards.
// Every lane of the wavefront must take part.
__device__ __forceinline__ void sum_runs(const Runs& r, float (&v)[4]) {
    run_step<1>(v, r.take[0]);
    run_step<2>(v, r.take[1]);
    run_step<4>(v, r.take[2]);
    run_step<8>(v, r.take[3]);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float part = dpp<kRowBcast15>(v[k]);
        if (r.takes_offer) v[k] += part;
    }
}

constexpr int kLineSlots = 128;   // lines per wavefront's table
constexpr int kLineProbes = 4;
constexpr int kLineRest = 7;
constexpr uint32_t kLineFree = 0xFFFFFFFFu;
// float k of slot h sits at k * kLinePitch + h: the sixteen floats of a line
// and the same float of neighbouring slots fall into different banks
constexpr int kLinePitch = kLineSlots + 1;

struct LineTable {
    float val[16 * kLinePitch];
    uint32_t key[kLineSlots];
    // rows on their way to memory without the table; the flush keeps its list
    // of used slots in the same place
    union {
        struct {
            uint32_t row[64];
            float v[64 * 4];
        } out;
        uint32_t used[kLineSlots];
    };
};

// Orders the LDS traffic of one wavefront (whose LDS instructions execute in
// program order, each for all its lanes) for the compiler.
__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// at[k * kLinePitch] += v[k], k = 0..3, in LDS.  The LDS executes a
// floating-point add atomic one lane after the other (about three cycles a
// lane, measured) and a 32-bit compare-and-swap at full rate: the add is a read
// and a compare-and-swap of the sum.  The four floats go side by side, two
// round trips for all of them; lanes that met another lane's update in between
// (seldom: runs of equal rows have been summed before) repeat float by float.
__device__ __forceinline__ void lds_add4(float* at, const float (&v)[4]) {
    unsigned int* w = reinterpret_cast<unsigned int*>(at);
    unsigned int seen[4], got[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) seen[k] = w[k * kLinePitch];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        got[k] = atomicCAS(w + k * kLinePitch, seen[k],
                           __float_as_uint(__uint_as_float(seen[k]) + v[k]));
    }
    if (got[0] == seen[0] && got[1] == seen[1] && got[2] == seen[2] && got[3] == seen[3]) return;
#pragma unroll 1
    for (int k = 0; k < 4; ++k) {
        // (selects, not an indexed access: the arrays stay in registers)
        unsigned int g = k == 0 ? got[0] : k == 1 ? got[1] : k == 2 ? got[2] : got[3];
        unsigned int s = k == 0 ? seen[0] : k == 1 ? seen[1] : k == 2 ? seen[2] : seen[3];
        const float add = k == 0 ? v[0] : k == 1 ? v[1] : k == 2 ? v[2] : v[3];
        while (g != s) {
            s = g;
            g = atomicCAS(w + k * kLinePitch, s, __float_as_uint(__uint_as_float(s) + add));
        }
    }
}

struct LineAcc {
    LineTable* tab;
    int rest;      // tiles left during which the table is left aside
    int spilled;   // rows that found no place in the table since the last flush (whole wavefront)

    __device__ __forceinline__ void start(LineTable* t, int lane) {
        tab = t;
        rest = 0;
        spilled = 0;
        if (tab != nullptr) {
            for (int i = lane; i < 16 * kLinePitch; i += 64) tab->val[i] = 0.f;
            tab->key[lane] = kLineFree;
            tab->key[lane + 64] = kLineFree;
            wave_lds_fence();
        }
    }

    // grad[4 * row .. 4 * row + 3] += v for the lanes that `want`; every lane
    // of the wavefront must take part.
    __device__ __forceinline__ void add4(float* __restrict__ grad, bool want, uint32_t row,
                                         const float (&v)[4], int lane) {
        bool placed = false;
        if (want && rest == 0) {
            const uint32_t line = row >> 2;
            uint32_t h = (line * 0x9E3779B1u) >> 25;
#pragma unroll 1
            for (int p = 0; p < kLineProbes; ++p) {
                const uint32_t old = atomicCAS(&tab->key[h], kLineFree, line);
                if (old == kLineFree || old == line) {
                    placed = true;
                    break;
                }
                h = (h + 1) & (kLineSlots - 1);
            }
            if (placed) lds_add4(tab->val + (row & 3u) * 4 * kLinePitch + h, v);
        }
        // The rest goes to memory now, regrouped so that the four floats of a
        // row leave from neighbouring lanes of one instruction (one request a
        // row; one lane sending its four floats would make four).
        const uint64_t out = __ballot(want && !placed);
        if (out == 0) return;
        const int n = __popcll(out);
        spilled += n;
        wave_lds_fence();
        if (want && !placed) {
            const int at = __popcll(out & ((1ull << lane) - 1ull));
            tab->out.row[at] = row;
            *reinterpret_cast<float4*>(tab->out.v + at * 4) = make_float4(v[0], v[1], v[2], v[3]);
        }
        wave_lds_fence();
        for (int i = 0; i < n; i += 16) {
            const int e = i + (lane >> 2);
            if (e < n) {
                unsafeAtomicAdd(grad + static_cast<uint64_t>(tab->out.row[e]) * 4 + (lane & 3),
                                tab->out.v[e * 4 + (lane & 3)]);
            }
        }
        wave_lds_fence();
    }

    // Whole wavefront: sends the table's lines out and empties it.
    __device__ __forceinline__ void flush(float* __restrict__ grad, int lane) {
        if (rest > 0) {
            --rest;
        } else {
            wave_lds_fence();
            const bool lo = tab->key[lane] != kLineFree;
            const bool hi = tab->key[lane + 64] != kLineFree;
            const uint64_t mlo = __ballot(lo), mhi = __ballot(hi);
            const uint64_t below = (1ull << lane) - 1ull;
            const int nlo = __popcll(mlo);
            const int n = nlo + __popcll(mhi);
            if (lo) tab->used[__popcll(mlo & below)] = lane;
            if (hi) tab->used[nlo + __popcll(mhi & below)] = lane + 64;
            wave_lds_fence();
            // four lines per instruction, sixteen lines per turn: the reads of
            // a turn are issued together
            for (int i = 0; i < n; i += 16) {
                uint32_t h[4], line[4];
                float v[4];
                float* at[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int e = i + j * 4 + (lane >> 4);
                    h[j] = e < n ? tab->used[e] : 0u;
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int e = i + j * 4 + (lane >> 4);
                    at[j] = tab->val + (lane & 15) * kLinePitch + h[j];
                    line[j] = tab->key[h[j]];
                    v[j] = e < n ? *at[j] : 0.f;
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    // floats nobody contributed to are zero
                    if (v[j] != 0.f) {
                        *at[j] = 0.f;
                        unsafeAtomicAdd(
                                grad + ((static_cast<uint64_t>(line[j]) << 4) | (lane & 15)), v[j]);
                    }
                }
            }
            wave_lds_fence();
            tab->key[lane] = kLineFree;
            tab->key[lane + 64] = kLineFree;
            wave_lds_fence();
            // more rows went past the table than it has lines
            if (spilled > kLineSlots) rest = kLineRest;
        }
        spilled = 0;
    }
};

// grad_emb[row, 0..3] += v for the lanes that are `on`; every lane of the
// wavefront must take part.  `runs`: find_runs of this tile.
__device__ __forceinline__ void accumulate_row4(LineAcc& acc, float* __restrict__ grad_emb,
                                                uint32_t row, bool on, const Runs& runs,
                                                float (&v)[4], int lane) {
    bool tail = true;
    if (runs.any) {   // (samples cells apart, scattered points: nothing to join)
        sum_runs(runs, v);
        tail = runs.tail;
    }
    acc.add4(grad_emb, on && tail, row, v, lane);
}

// The runs of a tile: lanes without a query get a number no neighbour shares.
__device__ __forceinline__ Runs tile_runs(uint32_t cell_row, bool on, int lane) {
    return find_runs(on ? cell_row : (kNoRow - static_cast<uint32_t>(lane & 1)), lane);
}

__device__ __forceinline__ LineTable* line_table(unsigned char* smem, const QDev& a,
                                                 bool lds_lut, bool wanted) {
    if (!wanted) return nullptr;
    return reinterpret_cast<LineTable*>(smem + table_offset(a, 1, lds_lut)) +
           (threadIdx.x >> 6);
}

// First-order backward, E = 4 (formulas as in query_backward_forward_kernel).
template <bool LDS, int OUT>
__global__ __launch_bounds__(kBlock, kWavesWide) void
query_backward_forward_vec_kernel(
        QDev a, const float* __restrict__ z, float* __restrict__ grad_emb,
        float* __restrict__ grad_off) {
    extern __shared__ __align__(16) unsigned char smem[];
    const CellLut lut = stage_cell_lut<LDS>(a, smem);
    const int lane = threadIdx.x & 63;
    const float* __restrict__ emb = static_cast<const float*>(a.emb);
    constexpr bool want_emb = (OUT & 1) != 0;
    constexpr bool want_off = (OUT & 2) != 0;
    LineAcc acc;
    acc.start(line_table(smem, a, LDS, want_emb), lane);
    const int64_t ntiles = (a.N + kBlock - 1) / kBlock;
    TileWalk walk(ntiles);
    for (int64_t tile = walk.next; tile < walk.end; tile += walk.step) {
        uint32_t row[8];
        float o[3];
        const int64_t q = tile * kBlock + threadIdx.x;
        const QueryInputs in = load_inputs(a, q);
        resolve_rows<LDS>(a, lut, in, row, o);
        const bool on = row[0] != kNoRow;
        float4 z4 = make_float4(0.f, 0.f, 0.f, 0.f);
        if (on) {
            typedef float v4f __attribute__((ext_vector_type(4)));
            const v4f zl = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(z + q * 4));
            z4 = make_float4(zl.x, zl.y, zl.z, zl.w);
        }
        AxisTerms<float> t;
        axis_terms<float, true>(o, a.smooth, t);
        // the gathered rows are used up before the scatter starts, which keeps
        // them out of the registers the scatter needs
        if constexpr (want_off) {
            float4 e[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                e[c] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (on) {
                    e[c] = *reinterpret_cast<const float4*>(
                            emb + static_cast<int64_t>(row[c]) * 4);
                }
            }
            float go[3] = {0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                float gw[3];
                corner_weight_grad<float>(t, c, gw);
                float dot = e[c].x * z4.x;
                dot += e[c].y * z4.y;
                dot += e[c].z * z4.z;
                dot += e[c].w * z4.w;
                go[0] += dot * gw[0];
                go[1] += dot * gw[1];
                go[2] += dot * gw[2];
            }
            if (q < a.N) {
                __builtin_nontemporal_store(on ? go[0] : 0.f, grad_off + q * 3 + 0);
                __builtin_nontemporal_store(on ? go[1] : 0.f, grad_off + q * 3 + 1);
                __builtin_nontemporal_store(on ? go[2] : 0.f, grad_off + q * 3 + 2);
            }
        }
        if constexpr (want_emb) {
            const Runs runs = tile_runs(row[0], on, lane);
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const float w = corner_weight<float>(t, c);
                float v[4] = {w * z4.x, w * z4.y, w * z4.z, w * z4.w};
                accumulate_row4(acc, grad_emb, row[c], on, runs, v, lane);
            }
            acc.flush(grad_emb, lane);
        }
    }
}

// Backward of the backward, E = 4 (formulas as in
// query_backward_backward_kernel).
template <bool LDS, int OUT>
__global__ __launch_bounds__(kBlock, kWavesWide) void
query_backward_backward_vec_kernel(
        QDev a, const float* __restrict__ gg_off, const float* __restrict__ z,
        float* __restrict__ grad_z, float* __restrict__ grad_emb) {
    extern __shared__ __align__(16) unsigned char smem[];
    const CellLut lut = stage_cell_lut<LDS>(a, smem);
    const int lane = threadIdx.x & 63;
    const float* __restrict__ emb = static_cast<const float*>(a.emb);
    constexpr bool want_emb = (OUT & 1) != 0;
    constexpr bool want_z = (OUT & 2) != 0;
    LineAcc acc;
    acc.start(line_table(smem, a, LDS, want_emb), lane);
    const int64_t ntiles = (a.N + kBlock - 1) / kBlock;
    TileWalk walk(ntiles);
    for (int64_t tile = walk.next; tile < walk.end; tile += walk.step) {
        uint32_t row[8];
        float o[3];
        const int64_t q = tile * kBlock + threadIdx.x;
        const QueryInputs in = load_inputs(a, q);
        resolve_rows<LDS>(a, lut, in, row, o);
        const bool on = row[0] != kNoRow;
        float4 z4 = make_float4(0.f, 0.f, 0.f, 0.f);
        float gg[3] = {0.f, 0.f, 0.f};
        if (on) {
            typedef float v4f __attribute__((ext_vector_type(4)));
            const v4f zl = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(z + q * 4));
            z4 = make_float4(zl.x, zl.y, zl.z, zl.w);
            gg[0] = __builtin_nontemporal_load(gg_off + q * 3 + 0);
            gg[1] = __builtin_nontemporal_load(gg_off + q * 3 + 1);
            gg[2] = __builtin_nontemporal_load(gg_off + q * 3 + 2);
        }
        AxisTerms<float> t;
        axis_terms<float, true>(o, a.smooth, t);
        if constexpr (want_z) {
            float4 e[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                e[c] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (on) {
                    e[c] = *reinterpret_cast<const float4*>(
                            emb + static_cast<int64_t>(row[c]) * 4);
                }
            }
            float gz[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                float gw[3];
                corner_weight_grad<float>(t, c, gw);
                const float d = gw[0] * gg[0] + gw[1] * gg[1] + gw[2] * gg[2];
                gz[0] += d * e[c].x;
                gz[1] += d * e[c].y;
                gz[2] += d * e[c].z;
                gz[3] += d * e[c].w;
            }
            if (q < a.N) {
                typedef float v4f __attribute__((ext_vector_type(4)));
                const v4f g4 = {on ? gz[0] : 0.f, on ? gz[1] : 0.f, on ? gz[2] : 0.f, on ? gz[3] : 0.f};
                __builtin_nontemporal_store(g4, reinterpret_cast<v4f*>(grad_z + q * 4));
            }
        }
        if constexpr (want_emb) {
            const Runs runs = tile_runs(row[0], on, lane);
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                float gw[3];
                corner_weight_grad<float>(t, c, gw);
                const float d = gw[0] * gg[0] + gw[1] * gg[1] + gw[2] * gg[2];
                float v[4] = {d * z4.x, d * z4.y, d * z4.z, d * z4.w};
                accumulate_row4(acc, grad_emb, row[c], on, runs, v, lane);
            }
            acc.flush(grad_emb, lane);
        }
    }
}

// Sparse convolution forward (ash/src/grid.cu:948-1043): for every cell of the
// listed blocks, out[row] = sum over the K window taps k of
// in[row of neighbour k] * w[k], channel by channel, taps whose block is
// missing skipped.  One lane per (cell, channel): a wavefront reads whole rows
// of neighbouring cells, and the taps are accumulated in the reference's order
// with one fused multiply-add each (what nvcc makes of `sum += in * w`).
struct ConvDev {
    const void* in;
    const void* w;
    const uint8_t* masks;
    const int64_t* grid_indices;
    const int64_t* cell_indices;
    const int64_t* lut_g;     // [B, GN]
    const int64_t* lut_c2c;   // [M, K]
    const int64_t* lut_c2g;   // [M, K]
    void* out;
    int64_t n_grids, B, M, E, K, GN;
    int owns;   // the kernel writes every cell of the listed blocks (zeros where it has no result)
};

// One lane per cell with all channels of the row in registers (EC >= E, a
// power of two up to 16): consecutive lanes are consecutive cells, so a tap
// reads a contiguous run of rows, and the table entries are fetched once per
// cell instead of once per channel.  `vec4`: fp32 rows of a multiple of four
// channels on 16-byte aligned buffers are moved as float4.
template <typename T, int EC>
__global__ __launch_bounds__(kBlock) void convolution_cell_kernel(ConvDev a, int vec4) {
    const int64_t item = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (item >= a.n_grids * a.M || !a.masks[item]) return;
    const int64_t g = a.grid_indices[item / a.M];
    const int64_t c = a.cell_indices[item % a.M];
    if (g < 0 || g >= a.B || c < 0 || c >= a.M) return;
    const T* in = static_cast<const T*>(a.in);
    const T* w = static_cast<const T*>(a.w);
    const int64_t* nb_g = a.lut_g + g * a.GN;
    const int64_t* nb_c = a.lut_c2c + c * a.K;
    const int64_t* nb_n = a.lut_c2g + c * a.K;
    const int E = static_cast<int>(a.E);
    T acc[EC];
#pragma unroll
    for (int e = 0; e < EC; ++e) acc[e] = T(0);
    for (int64_t k = 0; k < a.K; ++k) {
        const int64_t gn = nb_n[k];
        if (gn < 0 || gn >= a.GN) continue;
        const int64_t gi = nb_g[gn];
        if (gi < 0 || gi >= a.B) continue;
        const int64_t ci = nb_c[k];
        if (ci < 0 || ci >= a.M) continue;
        const T* row = in + (gi * a.M + ci) * E;
        const T* wk = w + k * E;
        if constexpr (sizeof(T) == 4 && EC >= 4) {
            if (vec4) {
#pragma unroll
                for (int q = 0; q < EC / 4; ++q) {
                    if (4 * q < E) {
                        const float4 r = reinterpret_cast<const float4*>(row)[q];
                        acc[4 * q + 0] = fmaf(r.x, wk[4 * q + 0], acc[4 * q + 0]);
                        acc[4 * q + 1] = fmaf(r.y, wk[4 * q + 1], acc[4 * q + 1]);
                        acc[4 * q + 2] = fmaf(r.z, wk[4 * q + 2], acc[4 * q + 2]);
                        acc[4 * q + 3] = fmaf(r.w, wk[4 * q + 3], acc[4 * q + 3]);
                    }
                }
                continue;
            }
        }
#pragma unroll
        for (int e = 0; e < EC; ++e) {
            if (e < E) acc[e] = fma(row[e], wk[e], acc[e]);
        }
    }
    T* o = static_cast<T*>(a.out) + (g * a.M + c) * E;
    if constexpr (sizeof(T) == 4 && EC >= 4) {
        if (vec4) {
#pragma unroll
            for (int q = 0; q < EC / 4; ++q) {
                if (4 * q < E) {
                    reinterpret_cast<float4*>(o)[q] = make_float4(
                            acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]);
                }
            }
            return;
        }
    }
#pragma unroll
    for (int e = 0; e < EC; ++e) {
        if (e < E) o[e] = acc[e];
    }
}

// The same per-cell accumulation with one persistent workgroup per block of
// cells at a time: the block's own rows are staged in LDS (for a 3^3 window
// about four taps in five stay inside the block) and the two per-cell tables
// are kept in LDS in compact form (uint16 cell, uint8 block offset) for the
// whole launch, when they fit.  Taps, order and arithmetic are unchanged.
constexpr int kConvThreads = 512;
unsigned persistent_grid(int64_t ntiles, size_t smem, int max_per_cu = 8);

template <typename T, int EC>
__global__ __launch_bounds__(kConvThreads) void convolution_block_kernel(
        ConvDev a, int vec4, int lut_lds, int rows_lds) {
    extern __shared__ __align__(16) unsigned char conv_smem[];
    const int tid = threadIdx.x;
    const int E = static_cast<int>(a.E);
    const int M = static_cast<int>(a.M);
    const int K = static_cast<int>(a.K);
    T* rows = reinterpret_cast<T*>(conv_smem);
    const size_t rows_bytes =
            rows_lds ? (static_cast<size_t>(M) * E * sizeof(T) + 15) / 16 * 16 : 0;
    uint16_t* cc = reinterpret_cast<uint16_t*>(conv_smem + rows_bytes);
    uint8_t* cg = reinterpret_cast<uint8_t*>(cc + static_cast<size_t>(M) * K);
    if (lut_lds) {
        for (int t = tid; t < M * K; t += kConvThreads) {
            const int64_t ci = a.lut_c2c[t];
            const int64_t gn = a.lut_c2g[t];
            cc[t] = (ci >= 0 && ci < M) ? static_cast<uint16_t>(ci) : 0xFFFFu;
            cg[t] = (gn >= 0 && gn < a.GN) ? static_cast<uint8_t>(gn) : 0xFFu;
        }
    }
    const T* in = static_cast<const T*>(a.in);
    const T* w = static_cast<const T*>(a.w);
    for (int64_t blk = blockIdx.x; blk < a.n_grids; blk += gridDim.x) {
        const int64_t g = a.grid_indices[blk];
        const bool g_ok = g >= 0 && g < a.B;
        __syncthreads();
        if (rows_lds && g_ok) {
            const T* src = in + g * a.M * E;
            if (vec4) {
                for (int t = tid; t < M * E / 4; t += kConvThreads) {
                    reinterpret_cast<float4*>(rows)[t] = reinterpret_cast<const float4*>(src)[t];
                }
            } else {
                for (int t = tid; t < M * E; t += kConvThreads) rows[t] = src[t];
            }
        }
        __syncthreads();
        if (!g_ok) continue;
        const int64_t* nb_g = a.lut_g + g * a.GN;
        for (int c_i = tid; c_i < M; c_i += kConvThreads) {
            if (!a.masks[blk * a.M + c_i]) continue;
            const int64_t c = a.cell_indices[c_i];
            if (c < 0 || c >= a.M) continue;
            T acc[EC];
#pragma unroll
            for (int e = 0; e < EC; ++e) acc[e] = T(0);
            for (int k = 0; k < K; ++k) {
                int64_t gn, ci;
                if (lut_lds) {
                    const uint16_t ci16 = cc[c * K + k];
                    const uint8_t gn8 = cg[c * K + k];
                    if (ci16 == 0xFFFFu || gn8 == 0xFFu) continue;
                    ci = ci16;
                    gn = gn8;
                } else {
                    gn = a.lut_c2g[c * K + k];
                    ci = a.lut_c2c[c * K + k];
                    if (gn < 0 || gn >= a.GN || ci < 0 || ci >= a.M) continue;
                }
                const int64_t gi = nb_g[gn];
                if (gi < 0 || gi >= a.B) continue;
                const T* row = (rows_lds && gi == g) ? rows + ci * E
                                                     : in + (gi * a.M + ci) * E;
                const T* wk = w + static_cast<int64_t>(k) * E;
                if constexpr (sizeof(T) == 4 && EC >= 4) {
                    if (vec4) {
#pragma unroll
                        for (int q = 0; q < EC / 4; ++q) {
                            if (4 * q < E) {
                                const float4 r = reinterpret_cast<const float4*>(row)[q];
                                acc[4 * q + 0] = fmaf(r.x, wk[4 * q + 0], acc[4 * q + 0]);
                                acc[4 * q + 1] = fmaf(r.y, wk[4 * q + 1], acc[4 * q + 1]);
                                acc[4 * q + 2] = fmaf(r.z, wk[4 * q + 2], acc[4 * q + 2]);
                                acc[4 * q + 3] = fmaf(r.w, wk[4 * q + 3], acc[4 * q + 3]);
                            }
                        }
                        continue;
                    }
                }
#pragma unroll
                for (int e = 0; e < EC; ++e) {
                    if (e < E) acc[e] = fma(row[e], wk[e], acc[e]);
                }
            }
            T* o = static_cast<T*>(a.out) + (g * a.M + c) * E;
            bool stored = false;
            if constexpr (sizeof(T) == 4 && EC >= 4) {
                if (vec4) {
#pragma unroll
                    for (int q = 0; q < EC / 4; ++q) {
                        if (4 * q < E) {
                            reinterpret_cast<float4*>(o)[q] = make_float4(
                                    acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]);
                        }
                    }
                    stored = true;
                }
            }
            if (!stored) {
#pragma unroll
                for (int e = 0; e < EC; ++e) {
                    if (e < E) o[e] = acc[e];
                }
            }
        }
    }
}

template <typename T, int EC>
int launch_convolution_block(const ConvDev& a, int vec4, hipStream_t s) {
    const size_t rows_bytes = (static_cast<size_t>(a.M) * a.E * sizeof(T) + 15) / 16 * 16;
    const size_t lut_bytes = static_cast<size_t>(a.M) * a.K * 3;
    const int rows_lds = rows_bytes <= 64 * 1024 ? 1 : 0;
    const int lut_lds = (lut_bytes <= 48 * 1024 && a.M < 0xFFFF && a.GN < 0xFF) ? 1 : 0;
    const size_t smem = (rows_lds ? rows_bytes : 0) + (lut_lds ? lut_bytes : 0) + 16;
    auto kernel = convolution_block_kernel<T, EC>;
    ASH_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(smem)));
    unsigned g = persistent_grid(a.n_grids, smem);
    kernel<<<g, kConvThreads, smem, s>>>(a, vec4, lut_lds, rows_lds);
    ASH_LAUNCH_CHECK();
    return 0;
}

// Cube windows over cubic blocks in the layout the Python layer builds
// (cell c = x + G y + G^2 z; tap k = (dx + r) + W (dy + r) + W^2 (dz + r) with
// W = 2 r + 1; neighbour block (bx + 1) + 3 (by + 1) + 9 (bz + 1)): the block's
// cells together with their halo of r cells, (G + 2r)^3 rows of EC channels,
// are staged in LDS once per block, and every cell then reads its W^3 taps from
// there -- in table order, one fused multiply-add per tap and channel, like the
// other kernels.  Rows of missing blocks are staged as zeros: with finite
// weights adding 0 * w leaves the accumulator as it is (it starts at +0 and so
// never is -0), which is what skipping the tap does.  Every workgroup first
// checks the two per-cell tables against this layout and, should they describe
// something else, takes its blocks through the tables instead.
// EC: channels per pass; WT: window edge when it is 3, 5 or 7, else 0; NY: cells
// per lane along y (0: one lane = one cell with all EC channels).
// The second launch bound asks for four wavefronts per SIMD (two workgroups
// per CU, at most 128 registers) for all but the widest instances, which need
// more registers than that for their window.
template <typename T, int EC, int WT, int NY>
__global__ __launch_bounds__(kConvThreads, (EC >= 16 && NY >= 8) ? 2 : 4) void convolution_tile_kernel(
        ConvDev a, int G, int r, int e0, int ec, int vec, int Tz) {
    constexpr bool YB = NY > 0;   // NY cells that follow each other in y per lane
    extern __shared__ __align__(16) unsigned char conv_smem[];
    __shared__ int64_t s_nb[2][28];   // rows of 27 neighbour blocks + the block itself
    __shared__ int s_bad;
    const int tid = threadIdx.x;
    const int E = static_cast<int>(a.E);
    const int M = static_cast<int>(a.M);
    const int K = static_cast<int>(a.K);
    const int W = WT > 0 ? WT : 2 * r + 1;   // WT: window edge known at compile time
    const int Tn = G + 2 * r;
    const int T3 = Tn * Tn * Tn;
    // Tz: words from one z layer of a channel's plane to the next, Tn * Tn or
    // a little more (YB): the lanes of a wavefront read G words along x at
    // NY * Tn words from one group of lanes to the next in y and Tz in z, and
    // the host pads Tz so that the groups served together fall on different
    // LDS banks.
    const int Ts = Tz * Tn;        // words of one channel's plane
    const int zpad = Tz - Tn * Tn;
    T* tile = reinterpret_cast<T*>(conv_smem);                             // [Ts][EC]
    T* s_w = tile + static_cast<size_t>(Ts) * EC;                          // [K][EC]
    uint32_t* s_src = reinterpret_cast<uint32_t*>(s_w + static_cast<size_t>(K) * EC);  // [T3]
    uint16_t* s_inv = reinterpret_cast<uint16_t*>(s_src + T3);   // [M] position of a cell in cell_indices (YB)
    // YB keeps one plane per channel (a lane reads runs of one channel along
    // x), otherwise the channels of a row sit together.  p counts the rows of
    // the tile without the padding.
    auto plane_at = [&](int p) { return p + zpad * (p / (Tn * Tn)); };
    auto tile_at = [&](int p, int q) { return YB ? q * Ts + plane_at(p) : p * EC + q; };
    auto w_at = [&](int k, int q) { return YB ? q * K + k : k * EC + q; };
    const T* in = static_cast<const T*>(a.in);
    const T* w = static_cast<const T*>(a.w);
    T* out = static_cast<T*>(a.out);

    if (tid == 0) s_bad = 0;
    __syncthreads();
    {
        int bad = 0;
        for (int t = tid; t < M * K; t += kConvThreads) {
            const int c = t / K;
            const int k = t - c * K;
            const int x[3] = {c % G, (c / G) % G, c / (G * G)};
            const int o[3] = {k % W - r, (k / W) % W - r, k / (W * W) - r};
            int gn = 0, ci = 0, gs = 1, cs = 1;
#pragma unroll
            for (int d = 0; d < 3; ++d) {
                const int t_d = x[d] + o[d];
                const int b = t_d < 0 ? -1 : (t_d >= G ? 1 : 0);
                gn += (b + 1) * gs;
                ci += (t_d - b * G) * cs;
                gs *= 3;
                cs *= G;
            }
            bad |= a.lut_c2g[t] != gn || a.lut_c2c[t] != ci;
        }
        if (bad) s_bad = 1;
        // where every row of the tile comes from and where it goes:
        // place in the tile << 17 | neighbour block << 12 | cell
        for (int p = tid; p < T3; p += kConvThreads) {
            const int tx[3] = {p % Tn - r, (p / Tn) % Tn - r, p / (Tn * Tn) - r};
            int gn = 0, ci = 0, gs = 1, cs = 1;
#pragma unroll
            for (int d = 0; d < 3; ++d) {
                const int b = tx[d] < 0 ? -1 : (tx[d] >= G ? 1 : 0);
                gn += (b + 1) * gs;
                ci += (tx[d] - b * G) * cs;
                gs *= 3;
                cs *= G;
            }
            s_src[p] = (static_cast<uint32_t>(tile_at(p, 0)) << 17) | static_cast<uint32_t>((gn << 12) | ci);
        }
        for (int t = tid; t < K * EC; t += kConvThreads) {
            const int k = t / EC;
            const int q = t - k * EC;
            s_w[w_at(k, q)] = q < ec ? w[k * E + e0 + q] : T(0);
        }
        if constexpr (YB) {
            for (int c = tid; c < M; c += kConvThreads) s_inv[c] = 0xFFFFu;
        }
    }
    __syncthreads();
    if constexpr (YB) {
        for (int c_i = tid; c_i < M; c_i += kConvThreads) {
            const int64_t c = a.cell_indices[c_i];
            if (c >= 0 && c < a.M) s_inv[c] = static_cast<uint16_t>(c_i);
        }
    }
    __syncthreads();
    const bool by_table = s_bad != 0;

    // a.owns: nobody cleared the rows of the listed blocks, so cells without a
    // result get their zeros here.  The paths that visit cells through
    // cell_indices clear the whole block first, in the pass of the first
    // channels; the y-blocked path writes a zero where it skips a cell.
    auto clear_block = [&](int64_t g) {
        if (!a.owns || e0 != 0) return;
        T* rows = out + g * a.M * a.E;
        for (int64_t i = tid; i < a.M * a.E; i += kConvThreads) rows[i] = T(0);
        __syncthreads();
    };
    for (int64_t blk = blockIdx.x; by_table && blk < a.n_grids; blk += gridDim.x) {
        const int64_t g = a.grid_indices[blk];
        if (g < 0 || g >= a.B) continue;  // the same for the whole workgroup
        clear_block(g);
        {
            const int64_t* nb_g = a.lut_g + g * a.GN;
            for (int c_i = tid; c_i < M; c_i += kConvThreads) {
                if (!a.masks[blk * a.M + c_i]) continue;
                const int64_t c = a.cell_indices[c_i];
                if (c < 0 || c >= a.M) continue;
                T acc[EC];
#pragma unroll
                for (int q = 0; q < EC; ++q) acc[q] = T(0);
                for (int k = 0; k < K; ++k) {
                    const int64_t gn = a.lut_c2g[c * K + k];
                    if (gn < 0 || gn >= a.GN) continue;
                    const int64_t gi = nb_g[gn];
                    if (gi < 0 || gi >= a.B) continue;
                    const int64_t ci = a.lut_c2c[c * K + k];
                    if (ci < 0 || ci >= a.M) continue;
#pragma unroll
                    for (int q = 0; q < EC; ++q) {
                        if (q < ec) {
                            acc[q] = fma(in[(gi * a.M + ci) * E + e0 + q], s_w[w_at(k, q)], acc[q]);
                        }
                    }
                }
#pragma unroll
                for (int q = 0; q < EC; ++q) {
                    if (q < ec) out[(g * a.M + c) * E + e0 + q] = acc[q];
                }
            }
        }
    }
    if (by_table) return;

    // Blocks through the tile, software-pipelined: while a block is computed
    // from LDS, the rows of the next block's tile are already on their way
    // into registers and the row numbers of the block after that are fetched.
    // each XCD walks a contiguous eighth of the listing (TileWalk): with blocks
    // listed along a space-filling curve the halo rows are then mostly in the
    // XCD's own L2
    const TileWalk walk(a.n_grids);
    constexpr int kPre = EC >= 16 ? 2 : (EC >= 8 ? 4 : 6);   // tile rows a thread can hold
    const bool prefetch = T3 <= kPre * kConvThreads;
    auto fetch_rows = [&](int64_t b) -> int64_t {  // lanes 0..26 neighbours, 27 the block
        if (tid > 27 || b >= walk.end) return -1;
        const int64_t g = a.grid_indices[b];
        if (g < 0 || g >= a.B) return -1;
        if (tid == 27) return g;
        const int64_t row = a.lut_g[g * 27 + tid];
        return (row >= 0 && row < a.B) ? row : -1;
    };
    // src_cell: an entry of s_src, or kNoRow for a thread without a row
    constexpr uint32_t kNoRow = 0xFFFFFFFFu;
    const T* in_e0 = in + e0;
    const uint32_t block_words = static_cast<uint32_t>(M * E);   // <= 4096 * 16
    auto load_row = [&](const int64_t* nb, uint32_t src_cell, T (&v)[EC]) {
#pragma unroll
        for (int q = 0; q < EC; ++q) v[q] = T(0);
        if (src_cell == kNoRow) return;
        const int64_t row = nb[(src_cell >> 12) & 31];
        if (row < 0) return;
        // row < B < 2^31: one 32 x 32 -> 64 bit product
        const T* src = in_e0 + (static_cast<uint64_t>(static_cast<uint32_t>(row)) * block_words +
                                (src_cell & 0xFFF) * static_cast<uint32_t>(E));
        if (vec) {   // EC is a multiple of four here
#pragma unroll
            for (int q4 = 0; q4 < (EC + 3) / 4; ++q4) {
                const float4 f = reinterpret_cast<const float4*>(src)[q4];
                v[(4 * q4) % EC] = f.x;
                v[(4 * q4 + 1) % EC] = f.y;
                v[(4 * q4 + 2) % EC] = f.z;
                v[(4 * q4 + 3) % EC] = f.w;
            }
        } else {
#pragma unroll
            for (int q = 0; q < EC; ++q) {
                if (q < ec) v[q] = src[q];
            }
        }
    };
    // One lane = one channel of NY cells that follow each other in y.  For
    // every (dz, dy) the W weights of the tap row are read once and used by all
    // NY cells, and the NY tile rows they meet stay in registers from one dy to
    // the next (row dy + j serves cell j), so that a step costs one new tile
    // row and one weight row for NY * W fused multiply-adds.  Every cell still
    // sees its taps in table order: dz, then dy, then dx.
    constexpr int kNy = NY > 0 ? NY : 4;
    const int yq_n = G / kNy;
    const int combos = G * yq_n * G;
    auto window_sums = [&](const T* plane, const T* wq, T (&acc)[kNy]) {
#pragma unroll
        for (int j = 0; j < kNy; ++j) acc[j] = T(0);
#pragma unroll 1
        for (int dz = 0; dz < WT; ++dz) {
            const T* pz = plane + Tz * dz;
            T win[kNy][WT > 0 ? WT : 1];
#pragma unroll
            for (int yy = 0; yy < kNy - 1; ++yy) {
#pragma unroll
                for (int dx = 0; dx < WT; ++dx) win[yy][dx] = pz[Tn * yy + dx];
            }
#pragma unroll
            for (int dy = 0; dy < WT; ++dy) {
#pragma unroll
                for (int dx = 0; dx < WT; ++dx) {
                    win[(dy + kNy - 1) & (kNy - 1)][dx] = pz[Tn * (dy + kNy - 1) + dx];
                }
                T wr[WT > 0 ? WT : 1];
#pragma unroll
                for (int dx = 0; dx < WT; ++dx) wr[dx] = wq[(dz * WT + dy) * WT + dx];
#pragma unroll
                for (int j = 0; j < kNy; ++j) {
#pragma unroll
                    for (int dx = 0; dx < WT; ++dx) {
                        acc[j] = fma(win[(dy + j) & (kNy - 1)][dx], wr[dx], acc[j]);
                    }
                }
            }
        }
    };
    // Results go out through LDS when a thread can hold all of its items' sums
    // until the tile is no longer read: the tile's space then takes them cell
    // by cell (rows padded by one word against bank conflicts) and whole output
    // rows are written by consecutive lanes.  Written one channel per lane
    // straight from the registers, a row reaches memory as EC separate 4-byte
    // pieces from different wavefronts, which more than doubles the bytes
    // written.  Pays for its two barriers with full rows of 16 channels and
    // with 3^3 windows; the wider windows of narrower rows need the registers
    // that would hold the results for their window.
    constexpr int kHold = 4;
    const bool staged = YB && (EC >= 16 || (WT == 3 && EC >= 4)) && combos * EC <= kHold * kConvThreads;
    T held[kHold][kNy];
    // staged: combos divides the workgroup size, so the items of a thread are
    // the same cells in channels task_q, task_q + task_qstep, ...
    const int task_qstep = staged ? kConvThreads / combos : 0;
    const int task_q = staged ? tid / combos : EC;
    int task_plane = 0, task_cell = 0;
    if (staged) {
        const int rem = tid - task_q * combos;
        const int x = rem % G;
        const int y0 = kNy * ((rem / G) % yq_n);
        const int z = rem / (G * yq_n);
        task_plane = x + Tn * y0 + Tz * z;
        task_cell = (x + G * y0 + G * G * z) * (EC + 1);
    }
    int64_t blk = walk.next;
    int buf = 0;
    int64_t rows_reg = fetch_rows(blk);
    if (tid <= 27) s_nb[0][tid] = rows_reg;
    rows_reg = fetch_rows(blk + walk.step);
    __syncthreads();
    // what does not change from block to block is read once: the source and the
    // place in the tile of the rows this thread stages
    T pre[kPre][EC];
    uint32_t pre_src[kPre];
#pragma unroll
    for (int i = 0; i < kPre; ++i) {
        const int p = tid + i * kConvThreads;
        pre_src[i] = (prefetch && p < T3) ? s_src[p] : kNoRow;
    }
    if (prefetch) {
#pragma unroll
        for (int i = 0; i < kPre; ++i) load_row(s_nb[0], pre_src[i], pre[i]);
    }
    for (; blk < walk.end; blk += walk.step, buf ^= 1) {
        __syncthreads();  // the previous block's tile has been read
        const int64_t g = s_nb[buf][27];
        if (prefetch) {
#pragma unroll
            for (int i = 0; i < kPre; ++i) {
                if (pre_src[i] != kNoRow) {
                    T* at = tile + (pre_src[i] >> 17);
#pragma unroll
                    for (int q = 0; q < EC; ++q) at[YB ? q * Ts : q] = pre[i][q];
                }
            }
        } else {
            for (int p = tid; p < T3; p += kConvThreads) {
                T v[EC];
                const uint32_t src_cell = s_src[p];
                load_row(s_nb[buf], src_cell, v);
                T* at = tile + (src_cell >> 17);
#pragma unroll
                for (int q = 0; q < EC; ++q) at[YB ? q * Ts : q] = v[q];
            }
        }
        if (tid <= 27) s_nb[buf ^ 1][tid] = rows_reg;
        __syncthreads();
        rows_reg = fetch_rows(blk + 2 * walk.step);
        if (prefetch && blk + walk.step < walk.end) {
#pragma unroll
            for (int i = 0; i < kPre; ++i) load_row(s_nb[buf ^ 1], pre_src[i], pre[i]);
        }
        if (g < 0) continue;  // the same for the whole workgroup
        if constexpr (YB) {
            if (staged) {
#pragma unroll
                for (int it = 0; it < kHold; ++it) {
                    const int q = task_q + it * task_qstep;
                    if (q < ec) window_sums(tile + q * Ts + task_plane, s_w + q * K, held[it]);
                }
                __syncthreads();  // the tile has been read
                T* stage = tile;  // [M][EC + 1]
#pragma unroll
                for (int it = 0; it < kHold; ++it) {
                    const int q = task_q + it * task_qstep;
                    if (q >= ec) continue;
#pragma unroll
                    for (int j = 0; j < kNy; ++j) {
                        stage[task_cell + q + j * G * (EC + 1)] = held[it][j];
                    }
                }
                __syncthreads();
                T* out_g = out + static_cast<uint64_t>(static_cast<uint32_t>(g)) * block_words + e0;
                const uint8_t* mask_b = reinterpret_cast<const uint8_t*>(a.masks) + blk * a.M;
                if (vec && ec == EC) {   // whole rows, 16 bytes per lane
                    if constexpr (sizeof(T) == 4 && EC % 4 == 0) {
                        constexpr int kQ = EC / 4;
                        for (int i = tid; i < M * kQ; i += kConvThreads) {
                            const int c = i / kQ;
                            const int q4 = i - c * kQ;
                            const int c_i = s_inv[c];
                            const bool keep = c_i != 0xFFFF && mask_b[c_i];
                            if (!keep && !a.owns) continue;
                            const T* sp = stage + c * (EC + 1) + 4 * q4;
                            reinterpret_cast<float4*>(out_g + static_cast<uint32_t>(c) * E)[q4] =
                                    keep ? make_float4(sp[0], sp[1], sp[2], sp[3])
                                         : make_float4(0.f, 0.f, 0.f, 0.f);
                        }
                    }
                } else {
                    for (int i = tid; i < M * ec; i += kConvThreads) {
                        const int c = i / ec;
                        const int q = i - c * ec;
                        const int c_i = s_inv[c];
                        const bool keep = c_i != 0xFFFF && mask_b[c_i];
                        if (!keep && !a.owns) continue;
                        out_g[static_cast<uint32_t>(c) * E + q] = keep ? stage[c * (EC + 1) + q] : T(0);
                    }
                }
            } else {
#pragma unroll 1
                for (int at = tid; at < combos * EC; at += kConvThreads) {
                    const int q = at / combos;
                    if (q >= ec) continue;
                    const int rem = at - q * combos;
                    const int x = rem % G;
                    const int y0 = kNy * ((rem / G) % yq_n);
                    const int z = rem / (G * yq_n);
                    T acc[kNy];
                    window_sums(tile + static_cast<size_t>(q) * Ts + x + Tn * y0 + Tz * z,
                                s_w + static_cast<size_t>(q) * K, acc);
#pragma unroll
                    for (int j = 0; j < kNy; ++j) {
                        const int c = x + G * (y0 + j) + G * G * z;
                        const int c_i = s_inv[c];
                        const bool keep = c_i != 0xFFFF && a.masks[blk * a.M + c_i];
                        if (!keep && !a.owns) continue;
                        out[(g * a.M + c) * E + e0 + q] = keep ? acc[j] : T(0);
                    }
                }
            }
            continue;
        }
        clear_block(g);
        for (int c_i = tid; c_i < M; c_i += kConvThreads) {
            if (!a.masks[blk * a.M + c_i]) continue;
            const int64_t c64 = a.cell_indices[c_i];
            if (c64 < 0 || c64 >= a.M) continue;
            const int c = static_cast<int>(c64);
            // tile index of the tap (-r, -r, -r) of this cell
            const int base = c % G + Tn * ((c / G) % G) + Tn * Tn * (c / (G * G));
            T acc[EC];
#pragma unroll
            for (int q = 0; q < EC; ++q) acc[q] = T(0);
            // only the innermost loop is unrolled: a fully unrolled window keeps
            // hundreds of values in flight and costs the occupancy
#pragma unroll 1
            for (int dz = 0; dz < W; ++dz) {
#pragma unroll 1
                for (int dy = 0; dy < W; ++dy) {
                    const T* row = tile + static_cast<size_t>(base + Tn * dy + Tn * Tn * dz) * EC;
                    const T* wrow = s_w + static_cast<size_t>((dz * W + dy) * W) * EC;
                    if constexpr (WT > 0) {
#pragma unroll
                        for (int dx = 0; dx < WT; ++dx) {
#pragma unroll
                            for (int q = 0; q < EC; ++q) {
                                acc[q] = fma(row[dx * EC + q], wrow[dx * EC + q], acc[q]);
                            }
                        }
                    } else {
                        for (int dx = 0; dx < W; ++dx) {
#pragma unroll
                            for (int q = 0; q < EC; ++q) {
                                acc[q] = fma(row[dx * EC + q], wrow[dx * EC + q], acc[q]);
                            }
                        }
                    }
                }
            }
#pragma unroll
            for (int q = 0; q < EC; ++q) {
                if (q < ec) out[(g * a.M + c) * E + e0 + q] = acc[q];
            }
        }
    }
}

// Settings of the tile kernel, each the fastest of the variants measured on
// 200 k blocks of 8^3 cells: windows from 27 taps on take the tile kernel, a
// tile may take 64 KB of LDS (two workgroups per CU), a lane handles four cells
// that follow each other in y (eight for windows of 5 and 7).
constexpr int kTileMinTaps = 27;
constexpr size_t kConvTileBytes = 64 * 1024;
constexpr bool kConvRowBlocking = true;
constexpr bool kConvRows8 = true;

// Largest cube edge G with G^3 == m, or 0.
inline int cube_edge(int64_t m) {
    int g = 1;
    while (static_cast<int64_t>(g) * g * g < m) ++g;
    return static_cast<int64_t>(g) * g * g == m ? g : 0;
}

// Takes the tile kernel when the sizes describe a cube window over cubic
// blocks with 27 neighbour blocks and the tile fits; returns -1 when not.
// `probe`: only say whether the tile kernel would take these sizes.
template <typename T>
int launch_convolution_tile(const ConvDev& a, hipStream_t s, bool probe = false) {
    const int G = cube_edge(a.M);
    const int W = cube_edge(a.K);
    if (G == 0 || W < 3 || W % 2 == 0 || a.GN != 27 || a.n_grids < 64) return -1;
    const int r = W / 2;
    if (r > G || a.M > 4096 || a.M * a.K > (int64_t{1} << 30)) return -1;
    const int64_t Tn = G + 2 * r;
    // cells per lane along y, as by_window below picks the instance
    const bool windowed = W == 3 || W == 5 || W == 7;
    const int ny = !(windowed && G % 4 == 0 && kConvRowBlocking) ? 0
                   : (G % 8 == 0 && kConvRows8 && W != 3) ? 8 : 4;
    // Words between the z layers of a channel's plane.  With blocks of 8^3 a
    // wavefront's lanes read 8 words along x per group, groups ny * Tn words
    // apart in y (four cells per lane) and one layer apart in z; the layers are
    // padded so that the four groups of every 32 lanes meet different banks.
    int64_t Tz = Tn * Tn;
    if (G == 8 && ny > 0 && sizeof(T) == 4) {
        const int a_y = static_cast<int>((4 * Tn) % 32);   // 8, 16 or 24
        int best = 32;
        for (int target : {8, 16, 24}) {
            const bool ok = ny == 8 ? target != 16 : (a_y == 16 ? target != 16 : target == 16);
            const int pad = static_cast<int>(((target - Tz) % 32 + 32) % 32);
            if (ok && pad < best) best = pad;
        }
        Tz += best;
    }
    // As many channels per pass as fit: a pass fetches the cache lines of all
    // channels of a row whatever it uses of them.
    constexpr int kMaxEc = sizeof(T) == 4 ? 16 : 8;
    const size_t cell_bytes = static_cast<size_t>(Tz * Tn) * sizeof(T);
    // two workgroups per CU (64 KB each) run faster than one with twice the
    // channels -- except for rows of a cache line or more, where every pass
    // over a part of the channels fetches the whole rows again: those may take
    // most of a CU's LDS for one workgroup (measured with 16 channels: 5^3
    // window in one pass 13.1 ms, in two passes of eight channels 15.5 ms)
    const size_t budget = a.E * sizeof(T) >= 64 ? 2 * kConvTileBytes : kConvTileBytes;
    int ec_max = kMaxEc;
    while (ec_max > 1 && cell_bytes * ec_max > budget) ec_max /= 2;
    if (cell_bytes * ec_max > budget) return -1;
    if (probe) return 0;
    const uintptr_t align = reinterpret_cast<uintptr_t>(a.in);
    for (int e0 = 0; e0 < a.E;) {
        int width = ec_max;                  // channels of the template instance
        while (width > 1 && width / 2 >= a.E - e0) width /= 2;
        const int ec = static_cast<int>(a.E - e0 < width ? a.E - e0 : width);
        const size_t smem = (cell_bytes + static_cast<size_t>(a.K) * sizeof(T)) * width +
                            static_cast<size_t>(Tn * Tn * Tn) * 4 + static_cast<size_t>(a.M) * 2 + 16;
        const int vec = (sizeof(T) == 4 && ec == width && width % 4 == 0 && a.E % 4 == 0 &&
                         e0 % 4 == 0 && align % 16 == 0) ? 1 : 0;
        const unsigned grid = persistent_grid(a.n_grids, smem + 512, 2048 / kConvThreads);
        auto launch = [&](auto kernel) -> int {
            ASH_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize,
                                        static_cast<int>(smem)));
            kernel<<<grid, kConvThreads, smem, s>>>(a, G, r, e0, ec, vec, static_cast<int>(Tz));
            ASH_LAUNCH_CHECK();
            return 0;
        };
        auto by_window = [&](auto ec_tag) -> int {
            constexpr int kEc = decltype(ec_tag)::value;
            if (G % 4 == 0 && kConvRowBlocking) {
                if (G % 8 == 0 && kConvRows8) {
                    if (W == 5) return launch(convolution_tile_kernel<T, kEc, 5, 8>);
                    if (W == 7) return launch(convolution_tile_kernel<T, kEc, 7, 8>);
                }
                if (W == 3) return launch(convolution_tile_kernel<T, kEc, 3, 4>);
                if (W == 5) return launch(convolution_tile_kernel<T, kEc, 5, 4>);
                if (W == 7) return launch(convolution_tile_kernel<T, kEc, 7, 4>);
            }
            if (W == 3) return launch(convolution_tile_kernel<T, kEc, 3, 0>);
            if (W == 5) return launch(convolution_tile_kernel<T, kEc, 5, 0>);
            if (W == 7) return launch(convolution_tile_kernel<T, kEc, 7, 0>);
            return launch(convolution_tile_kernel<T, kEc, 0, 0>);
        };
        int rc = 1;
        if (width == 16) {
            if constexpr (kMaxEc >= 16) rc = by_window(std::integral_constant<int, 16>());
        } else if (width == 8) {
            rc = by_window(std::integral_constant<int, 8>());
        } else if (width == 4) {
            rc = by_window(std::integral_constant<int, 4>());
        } else if (width == 2) {
            rc = by_window(std::integral_constant<int, 2>());
        } else {
            rc = by_window(std::integral_constant<int, 1>());
        }
        if (rc) return 1;
        e0 += ec;
    }
    return 0;
}

template <typename T>
int launch_convolution_cells(const ConvDev& a, hipStream_t s) {
    const int64_t threads = a.n_grids * a.M;
    const int64_t blocks = (threads + kBlock - 1) / kBlock;
    if (blocks > 0x7FFFFFFFll) ASH_FAIL("convolution_forward: too many cells in one call");
    const unsigned gb = static_cast<unsigned>(blocks);
    const uintptr_t align = reinterpret_cast<uintptr_t>(a.in) | reinterpret_cast<uintptr_t>(a.out);
    const int vec4 = (sizeof(T) == 4 && a.E % 4 == 0 && align % 16 == 0) ? 1 : 0;
    if (a.K >= kTileMinTaps) {
        const int rc = launch_convolution_tile<T>(a, s);
        if (rc >= 0) return rc;
    }
    if (a.n_grids >= 64 && a.M <= 4096) {
        // enough blocks to keep persistent workgroups busy
        if (a.E <= 1) return launch_convolution_block<T, 1>(a, vec4, s);
        if (a.E <= 2) return launch_convolution_block<T, 2>(a, vec4, s);
        if (a.E <= 4) return launch_convolution_block<T, 4>(a, vec4, s);
        if (a.E <= 8) return launch_convolution_block<T, 8>(a, vec4, s);
        return launch_convolution_block<T, 16>(a, vec4, s);
    }
    if (a.E <= 1) {
        convolution_cell_kernel<T, 1><<<gb, kBlock, 0, s>>>(a, vec4);
    } else if (a.E <= 2) {
        convolution_cell_kernel<T, 2><<<gb, kBlock, 0, s>>>(a, vec4);
    } else if (a.E <= 4) {
        convolution_cell_kernel<T, 4><<<gb, kBlock, 0, s>>>(a, vec4);
    } else if (a.E <= 8) {
        convolution_cell_kernel<T, 8><<<gb, kBlock, 0, s>>>(a, vec4);
    } else {
        convolution_cell_kernel<T, 16><<<gb, kBlock, 0, s>>>(a, vec4);
    }
    ASH_LAUNCH_CHECK();
    return 0;
}

// Wider rows than the reference supports (its accumulator holds 16 channels):
// one lane per (cell, channel).
template <typename T>
__global__ __launch_bounds__(kBlock) void convolution_forward_kernel(ConvDev a) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const int64_t item = t / a.E;
    const int e = static_cast<int>(t - item * a.E);
    if (item >= a.n_grids * a.M || !a.masks[item]) return;
    const int64_t g = a.grid_indices[item / a.M];
    const int64_t c = a.cell_indices[item % a.M];
    if (g < 0 || g >= a.B || c < 0 || c >= a.M) return;
    const T* in = static_cast<const T*>(a.in);
    const T* w = static_cast<const T*>(a.w);
    const int64_t* nb_g = a.lut_g + g * a.GN;
    const int64_t* nb_c = a.lut_c2c + c * a.K;
    const int64_t* nb_n = a.lut_c2g + c * a.K;
    T sum = T(0);
    for (int64_t k = 0; k < a.K; ++k) {
        const int64_t gn = nb_n[k];
        if (gn < 0 || gn >= a.GN) continue;
        const int64_t gi = nb_g[gn];
        if (gi < 0 || gi >= a.B) continue;
        const int64_t ci = nb_c[k];
        if (ci < 0 || ci >= a.M) continue;
        sum = fma(in[(gi * a.M + ci) * a.E + e], w[k * a.E + e], sum);
    }
    static_cast<T*>(a.out)[(g * a.M + c) * a.E + e] = sum;
}

__global__ __launch_bounds__(kBlock) void zero16_kernel(uint4* __restrict__ p,
                                                        int64_t n16) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    const uint4 v = make_uint4(0u, 0u, 0u, 0u);
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
         i < n16; i += stride) {
        p[i] = v;
    }
}

__global__ __launch_bounds__(kBlock) void zero1_kernel(
        unsigned char* __restrict__ p, int64_t n) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
         i < n; i += stride) {
        p[i] = 0;
    }
}

// listed[b] = 1 for every block of the listing.
__global__ __launch_bounds__(kBlock) void mark_listed_kernel(
        const int64_t* __restrict__ grid_indices, int64_t n, int64_t B,
        uint8_t* __restrict__ listed) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i >= n) return;
    const int64_t g = grid_indices[i];
    if (g >= 0 && g < B) listed[g] = 1;
}

// Zeroes the rows of the blocks that are not listed: `units` 16-byte pieces
// per block, one workgroup per block at a time.
__global__ __launch_bounds__(kBlock) void zero_unlisted_kernel(
        uint4* __restrict__ out, const uint8_t* __restrict__ listed, int64_t B,
        int64_t units) {
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    for (int64_t b = blockIdx.x; b < B; b += gridDim.x) {
        if (listed[b]) continue;  // the same for the whole workgroup
        uint4* rows = out + b * units;
        for (int64_t u = threadIdx.x; u < units; u += kBlock) rows[u] = zero;
    }
}

// ---------------------------------------------------------------- host
int zero_fill(void* ptr, int64_t bytes, hipStream_t s) {
    if (bytes <= 0) return 0;
    unsigned char* p = static_cast<unsigned char*>(ptr);
    // unaligned head
    const int64_t mis = (16 - reinterpret_cast<uintptr_t>(p) % 16) % 16;
    const int64_t head = mis < bytes ? mis : bytes;
    if (head > 0) {
        zero1_kernel<<<1, kBlock, 0, s>>>(p, head);
        ASH_LAUNCH_CHECK();
    }
    const int64_t n16 = (bytes - head) / 16;
    if (n16 > 0) {
        // one store per thread: workgroups handed out one after the other walk
        // through memory in order (6.8 TB/s; 5.7 with 16 384 workgroups striding)
        int64_t g = (n16 + kBlock - 1) / kBlock;
        if (g > 0x7FFFFFFF) g = 0x7FFFFFFF;
        zero16_kernel<<<static_cast<unsigned>(g), kBlock, 0, s>>>(
                reinterpret_cast<uint4*>(p + head), n16);
        ASH_LAUNCH_CHECK();
    }
    const int64_t tail = bytes - head - n16 * 16;
    if (tail > 0) {
        zero1_kernel<<<1, kBlock, 0, s>>>(p + head + n16 * 16, tail);
        ASH_LAUNCH_CHECK();
    }
    return 0;
}

// Runs of consecutive queries of a wavefront that meet the same row are summed
// before the atomic (2.4x faster on ray-ordered samples, neutral on shuffled
// ones); the kernels keep the plain variant as a template parameter.
constexpr bool merge_enabled() { return true; }

// `from_positions`: the per-query operand arrays are not read (the fused front
// end works them out), so they may be NULL.
int check_args(const ash_query_args* a, QDev& d, bool from_positions = false) {
    if (a == nullptr) ASH_FAIL("null query arguments");
    if (a->num_queries < 0) ASH_FAIL("negative query count");
    if (a->num_embeddings < 1 || a->cells_per_grid < 1) {
        ASH_FAIL("embeddings must have at least one block and one cell");
    }
    if (a->embedding_dim < 1 || a->embedding_dim > 16) {
        ASH_FAIL("embedding_dim must be in 1..16");
    }
    if (a->interpolation != ASH_INTERP_LINEAR &&
        a->interpolation != ASH_INTERP_SMOOTH_STEP) {
        ASH_FAIL("Unknown interpolation functor");
    }
    if (a->dtype != ASH_F32 && a->dtype != ASH_F64) ASH_FAIL("unknown dtype");
    if (a->num_embeddings > 0x7FFFFFFFll ||
        a->num_embeddings * a->cells_per_grid >= 0xFFFFFFFFll) {
        ASH_FAIL("num_embeddings * cells_per_grid must stay below 2^32 - 1");
    }
    if (a->embeddings == nullptr || a->lut_grid_nb2grid_idx == nullptr ||
        a->lut_cell_nb2cell_idx == nullptr || a->lut_cell_nb2grid_nb == nullptr) {
        ASH_FAIL("null table pointer");
    }
    if (a->num_queries > 0 && !from_positions &&
        (a->offsets == nullptr || a->grid_indices == nullptr ||
         a->cell_indices == nullptr || a->masks == nullptr)) {
        ASH_FAIL("null query pointer");
    }
    d.emb = a->embeddings;
    d.off = a->offsets;
    d.gidx = a->grid_indices;
    d.cidx = a->cell_indices;
    d.mask = a->masks;
    d.lut_g = a->lut_grid_nb2grid_idx;
    d.lut_c2c = a->lut_cell_nb2cell_idx;
    d.lut_c2g = a->lut_cell_nb2grid_nb;
    d.N = a->num_queries;
    d.B = a->num_embeddings;
    d.M = a->cells_per_grid;
    d.E = static_cast<int>(a->embedding_dim);
    d.smooth = a->interpolation == ASH_INTERP_SMOOTH_STEP ? 1 : 0;
    d.merge = merge_enabled() ? 1 : 0;
    return 0;
}

int pow2_ceil(int v) {
    int p = 1;
    while (p < v) p <<= 1;
    return p;
}

bool lut_in_lds(const QDev& d) { return d.M <= kMaxLdsCells; }

size_t smem_bytes(const QDev& d, int lpq, bool line_tables = false) {
    size_t bytes = table_offset(d, lpq, lut_in_lds(d));
    if (line_tables) bytes += (kBlock / 64) * sizeof(LineTable);
    return bytes;
}

// Enough persistent workgroups to fill every CU as far as LDS allows.
unsigned persistent_grid(int64_t ntiles, size_t smem, int max_per_cu) {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount,
                                  dev) == hipSuccess &&
            n > 0) {
            cus = n;
        } else {
            cus = 256;
        }
    }
    int per_cu = max_per_cu;
    if (smem > 0) {
        const int fit = static_cast<int>(kLdsPerCu / smem);
        if (fit < per_cu) per_cu = fit < 1 ? 1 : fit;
    }
    int64_t g = static_cast<int64_t>(cus) * per_cu;
    if (g > ntiles) g = ntiles;
    g = (g + kXcds - 1) / kXcds * kXcds;  // whole rounds over the XCDs
    if (g < kXcds) g = kXcds;
    return static_cast<unsigned>(g);
}

template <typename T, int VEC, int LPQ>
int launch_forward(const QDev& d, void* out, hipStream_t s) {
    const size_t smem = smem_bytes(d, LPQ);
    const unsigned g = persistent_grid((d.N + kBlock - 1) / kBlock, smem);
    if (lut_in_lds(d)) {
        query_forward_kernel<T, VEC, LPQ, true>
                <<<g, kBlock, smem, s>>>(d, static_cast<T*>(out));
    } else {
        query_forward_kernel<T, VEC, LPQ, false>
                <<<g, kBlock, smem, s>>>(d, static_cast<T*>(out));
    }
    ASH_LAUNCH_CHECK();
    return 0;
}

template <typename T, int VEC, int LPQ>
int launch_grid_forward(const QDev& d, const FrontDev& f, void* out, hipStream_t s) {
    const size_t smem = smem_bytes(d, LPQ);
    const unsigned g = persistent_grid((d.N + kBlock - 1) / kBlock, smem);
    const bool aux = f.gidx_out != nullptr;
#define ASH_GF(L, A)                                                          \
    grid_forward_kernel<T, VEC, LPQ, L, A><<<g, kBlock, smem, s>>>(d, f, static_cast<T*>(out))
    if (lut_in_lds(d)) {
        if (aux) ASH_GF(true, true);
        else ASH_GF(true, false);
    } else {
        if (aux) ASH_GF(false, true);
        else ASH_GF(false, false);
    }
#undef ASH_GF
    ASH_LAUNCH_CHECK();
    return 0;
}

template <typename T, int LPQ>
int launch_bwd_fwd(const QDev& d, const void* z, void* ge, void* go,
                   hipStream_t s) {
    const size_t smem = smem_bytes(d, LPQ);
    const unsigned g = persistent_grid((d.N + kBlock - 1) / kBlock, smem);
    const int out = (ge != nullptr ? 1 : 0) | (go != nullptr ? 2 : 0);
#define ASH_BF(L, O)                                                          \
    query_backward_forward_kernel<T, LPQ, L, O><<<g, kBlock, smem, s>>>(      \
            d, static_cast<const T*>(z), static_cast<T*>(ge),                 \
            static_cast<T*>(go))
    if (lut_in_lds(d)) {
        if (out == 3) ASH_BF(true, 3);
        else if (out == 1) ASH_BF(true, 1);
        else ASH_BF(true, 2);
    } else {
        if (out == 3) ASH_BF(false, 3);
        else if (out == 1) ASH_BF(false, 1);
        else ASH_BF(false, 2);
    }
#undef ASH_BF
    ASH_LAUNCH_CHECK();
    return 0;
}

template <typename T, int LPQ>
int launch_bwd_bwd(const QDev& d, const void* gg, const void* z, void* gz,
                   void* ge, hipStream_t s) {
    const size_t smem = smem_bytes(d, LPQ);
    const unsigned g = persistent_grid((d.N + kBlock - 1) / kBlock, smem);
    const int out = (ge != nullptr ? 1 : 0) | (gz != nullptr ? 2 : 0);
#define ASH_BB(L, O)                                                          \
    query_backward_backward_kernel<T, LPQ, L, O><<<g, kBlock, smem, s>>>(     \
            d, static_cast<const T*>(gg), static_cast<const T*>(z),           \
            static_cast<T*>(gz), static_cast<T*>(ge))
    if (lut_in_lds(d)) {
        if (out == 3) ASH_BB(true, 3);
        else if (out == 1) ASH_BB(true, 1);
        else ASH_BB(true, 2);
    } else {
        if (out == 3) ASH_BB(false, 3);
        else if (out == 1) ASH_BB(false, 1);
        else ASH_BB(false, 2);
    }
#undef ASH_BB
    ASH_LAUNCH_CHECK();
    return 0;
}

bool aligned16(const void* p) {
    return reinterpret_cast<uintptr_t>(p) % 16 == 0;
}

int launch_bwd_fwd_vec(const QDev& d, const void* z, void* ge, void* go,
                       hipStream_t s) {
    const size_t smem = smem_bytes(d, 1, ge != nullptr);
    const unsigned g = persistent_grid((d.N + kBlock - 1) / kBlock, smem);
    const int out = (ge != nullptr ? 1 : 0) | (go != nullptr ? 2 : 0);
#define ASH_BF(L, O)                                                          \
    query_backward_forward_vec_kernel<L, O><<<g, kBlock, smem, s>>>(     \
            d, static_cast<const float*>(z), static_cast<float*>(ge),         \
            static_cast<float*>(go))
    if (lut_in_lds(d)) {
        if (out == 3) ASH_BF(true, 3);
        else if (out == 1) ASH_BF(true, 1);
        else ASH_BF(true, 2);
    } else {
        if (out == 3) ASH_BF(false, 3);
        else if (out == 1) ASH_BF(false, 1);
        else ASH_BF(false, 2);
    }
#undef ASH_BF
    ASH_LAUNCH_CHECK();
    return 0;
}

int launch_bwd_bwd_vec(const QDev& d, const void* gg, const void* z, void* gz,
                       void* ge, hipStream_t s) {
    const size_t smem = smem_bytes(d, 1, ge != nullptr);
    const unsigned g = persistent_grid((d.N + kBlock - 1) / kBlock, smem);
    const int out = (ge != nullptr ? 1 : 0) | (gz != nullptr ? 2 : 0);
#define ASH_BB(L, O)                                                          \
    query_backward_backward_vec_kernel<L, O><<<g, kBlock, smem, s>>>(    \
            d, static_cast<const float*>(gg), static_cast<const float*>(z),   \
            static_cast<float*>(gz), static_cast<float*>(ge))
    if (lut_in_lds(d)) {
        if (out == 3) ASH_BB(true, 3);
        else if (out == 1) ASH_BB(true, 1);
        else ASH_BB(true, 2);
    } else {
        if (out == 3) ASH_BB(false, 3);
        else if (out == 1) ASH_BB(false, 1);
        else ASH_BB(false, 2);
    }
#undef ASH_BB
    ASH_LAUNCH_CHECK();
    return 0;
}

// fp32 rows of four channels on 16-byte aligned buffers
bool rows_as_float4(const QDev& d, const void* p0, const void* p1, const void* p2) {
    return d.E == 4 && aligned16(d.emb) && aligned16(p0) && aligned16(p1) &&
           aligned16(p2);
}

template <typename T>
int dispatch_forward(const QDev& d, void* out, hipStream_t s) {
    if constexpr (sizeof(T) == 4) {
        if (d.E % 4 == 0 && aligned16(d.emb) && aligned16(out)) {
            switch (d.E / 4) {
                case 1:
                    return launch_forward<float, 4, 1>(d, out, s);
                case 2:
                    return launch_forward<float, 4, 2>(d, out, s);
                default:
                    return launch_forward<float, 4, 4>(d, out, s);
            }
        }
    }
    if constexpr (sizeof(T) == 4) {
        // narrow rows that are not a multiple of four channels: one lane takes
        // the whole row (six channels: two lanes, three each), instead of one
        // lane per channel with a power of two of lanes per query
        switch (d.E) {
            case 2:
                return launch_forward<float, 2, 1>(d, out, s);
            case 3:
                return launch_forward<float, 3, 1>(d, out, s);
            case 5:
                return launch_forward<float, 5, 1>(d, out, s);
            case 6:
                return launch_forward<float, 3, 2>(d, out, s);
            default:
                break;
        }
    }
    switch (pow2_ceil(d.E)) {
        case 1:
            return launch_forward<T, 1, 1>(d, out, s);
        case 2:
            return launch_forward<T, 1, 2>(d, out, s);
        case 4:
            return launch_forward<T, 1, 4>(d, out, s);
        case 8:
            return launch_forward<T, 1, 8>(d, out, s);
        default:
            return launch_forward<T, 1, 16>(d, out, s);
    }
}

// Same choice of variant as dispatch_forward, so that the fused kernel adds up
// the corner rows in the same order as ash_query_forward on the same operands.
template <typename T>
int dispatch_grid_forward(const QDev& d, const FrontDev& f, void* out, hipStream_t s) {
    if constexpr (sizeof(T) == 4) {
        if (d.E % 4 == 0 && aligned16(d.emb) && aligned16(out)) {
            switch (d.E / 4) {
                case 1:
                    return launch_grid_forward<float, 4, 1>(d, f, out, s);
                case 2:
                    return launch_grid_forward<float, 4, 2>(d, f, out, s);
                default:
                    return launch_grid_forward<float, 4, 4>(d, f, out, s);
            }
        }
    }
    if constexpr (sizeof(T) == 4) {
        // narrow rows that are not a multiple of four channels: one lane takes
        // the whole row (six channels: two lanes, three each), instead of one
        // lane per channel with a power of two of lanes per query
        switch (d.E) {
            case 2:
                return launch_grid_forward<float, 2, 1>(d, f, out, s);
            case 3:
                return launch_grid_forward<float, 3, 1>(d, f, out, s);
            case 5:
                return launch_grid_forward<float, 5, 1>(d, f, out, s);
            case 6:
                return launch_grid_forward<float, 3, 2>(d, f, out, s);
            default:
                break;
        }
    }
    switch (pow2_ceil(d.E)) {
        case 1:
            return launch_grid_forward<T, 1, 1>(d, f, out, s);
        case 2:
            return launch_grid_forward<T, 1, 2>(d, f, out, s);
        case 4:
            return launch_grid_forward<T, 1, 4>(d, f, out, s);
        case 8:
            return launch_grid_forward<T, 1, 8>(d, f, out, s);
        default:
            return launch_grid_forward<T, 1, 16>(d, f, out, s);
    }
}

template <typename T>
int dispatch_bwd_fwd(const QDev& d, const void* z, void* ge, void* go,
                     hipStream_t s) {
    if constexpr (sizeof(T) == 4) {
        if (rows_as_float4(d, z, ge, nullptr)) return launch_bwd_fwd_vec(d, z, ge, go, s);
    }
    switch (pow2_ceil(d.E)) {
        case 1:
            return launch_bwd_fwd<T, 1>(d, z, ge, go, s);
        case 2:
            return launch_bwd_fwd<T, 2>(d, z, ge, go, s);
        case 4:
            return launch_bwd_fwd<T, 4>(d, z, ge, go, s);
        case 8:
            return launch_bwd_fwd<T, 8>(d, z, ge, go, s);
        default:
            return launch_bwd_fwd<T, 16>(d, z, ge, go, s);
    }
}

template <typename T>
int dispatch_bwd_bwd(const QDev& d, const void* gg, const void* z, void* gz,
                     void* ge, hipStream_t s) {
    if constexpr (sizeof(T) == 4) {
        if (rows_as_float4(d, z, ge, gz)) return launch_bwd_bwd_vec(d, gg, z, gz, ge, s);
    }
    switch (pow2_ceil(d.E)) {
        case 1:
            return launch_bwd_bwd<T, 1>(d, gg, z, gz, ge, s);
        case 2:
            return launch_bwd_bwd<T, 2>(d, gg, z, gz, ge, s);
        case 4:
            return launch_bwd_bwd<T, 4>(d, gg, z, gz, ge, s);
        case 8:
            return launch_bwd_bwd<T, 8>(d, gg, z, gz, ge, s);
        default:
            return launch_bwd_bwd<T, 16>(d, gg, z, gz, ge, s);
    }
}

int64_t elem_bytes(int dtype) { return dtype == ASH_F64 ? 8 : 4; }

}  // namespace
}  // namespace ash

using namespace ash;

extern "C" {

int ash_query_forward(const ash_query_args* a, void* output, void* stream) {
    QDev d;
    if (check_args(a, d)) return 1;
    if (d.N == 0) return 0;
    if (output == nullptr) ASH_FAIL("null output pointer");
    PointerGuard guard;
    ASH_HIP(guard.enter_for(a->embeddings));
    hipStream_t s = static_cast<hipStream_t>(stream);
    return a->dtype == ASH_F64 ? dispatch_forward<double>(d, output, s)
                               : dispatch_forward<float>(d, output, s);
}

int ash_grid_forward(ash_map_t* map, const float* x, const float* origin, float cell_size,
                     int grid_dim, const ash_query_args* tables, void* output, uint8_t* masks,
                     int64_t* grid_indices, int64_t* cell_indices, float* offsets,
                     void* stream) {
    if (map == nullptr) ASH_FAIL("null map handle");
    if (map->key_dim != 3) ASH_FAIL("grid queries need a map with 3-d keys");
    if (grid_dim < 1 || grid_dim > 1024) ASH_FAIL("grid_dim must be in 1..1024");
    if (!(cell_size > 0.f) || !(cell_size < INFINITY)) ASH_FAIL("cell_size must be positive and finite");
    QDev d;
    if (check_args(tables, d, true)) return 1;
    if (d.M != static_cast<int64_t>(grid_dim) * grid_dim * grid_dim) {
        ASH_FAIL("cells_per_grid must be grid_dim^3");
    }
    if (d.N > (int64_t{1} << 31) - kBlock) ASH_FAIL("too many positions in one call");
    if (d.N == 0) return 0;
    if (x == nullptr || output == nullptr || masks == nullptr) ASH_FAIL("null pointer");
    const int given = (grid_indices != nullptr) + (cell_indices != nullptr) + (offsets != nullptr);
    if (given != 0 && given != 3) {
        ASH_FAIL("grid_indices, cell_indices and offsets are written together: pass all or none");
    }
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (settle_table(map, s)) return 1;
    FrontDev f;
    f.m = map->d;
    f.x = x;
    f.origin = origin;
    f.inv_cell = 1.0f / cell_size;
    f.g = static_cast<float>(grid_dim);
    f.gdim = grid_dim;
    f.mask_out = masks;
    f.gidx_out = grid_indices;
    f.cidx_out = cell_indices;
    f.off_out = offsets;
    return tables->dtype == ASH_F64 ? dispatch_grid_forward<double>(d, f, output, s)
                                    : dispatch_grid_forward<float>(d, f, output, s);
}

namespace {

int backward_forward(const ash_query_args* a, const void* z, void* grad_embeddings,
                     void* grad_offsets, void* stream, bool clear) {
    QDev d;
    if (check_args(a, d)) return 1;
    if (grad_embeddings == nullptr && grad_offsets == nullptr) {
        ASH_FAIL("at least one of grad_embeddings / grad_offsets is required");
    }
    PointerGuard guard;
    ASH_HIP(guard.enter_for(a->embeddings));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (clear && grad_embeddings != nullptr &&
        zero_fill(grad_embeddings, d.B * d.M * d.E * elem_bytes(a->dtype), s)) {
        return 1;
    }
    if (d.N == 0) return 0;
    if (z == nullptr) ASH_FAIL("null pointer");
    return a->dtype == ASH_F64
                   ? dispatch_bwd_fwd<double>(d, z, grad_embeddings,
                                              grad_offsets, s)
                   : dispatch_bwd_fwd<float>(d, z, grad_embeddings,
                                             grad_offsets, s);
}

int backward_backward(const ash_query_args* a, const void* grad_grad_offsets,
                      const void* z, void* grad_z, void* grad_embeddings,
                      void* stream, bool clear) {
    QDev d;
    if (check_args(a, d)) return 1;
    if (grad_embeddings == nullptr && grad_z == nullptr) {
        ASH_FAIL("at least one of grad_z / grad_embeddings is required");
    }
    PointerGuard guard;
    ASH_HIP(guard.enter_for(a->embeddings));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (clear && grad_embeddings != nullptr &&
        zero_fill(grad_embeddings, d.B * d.M * d.E * elem_bytes(a->dtype), s)) {
        return 1;
    }
    if (d.N == 0) return 0;
    if (z == nullptr || grad_grad_offsets == nullptr) ASH_FAIL("null pointer");
    return a->dtype == ASH_F64
                   ? dispatch_bwd_bwd<double>(d, grad_grad_offsets, z, grad_z,
                                              grad_embeddings, s)
                   : dispatch_bwd_bwd<float>(d, grad_grad_offsets, z, grad_z,
                                             grad_embeddings, s);
}

}  // namespace

int ash_query_backward_forward(const ash_query_args* a, const void* z,
                               void* grad_embeddings, void* grad_offsets,
                               void* stream) {
    return backward_forward(a, z, grad_embeddings, grad_offsets, stream, true);
}

int ash_query_backward_forward_accumulate(const ash_query_args* a, const void* z,
                                          void* grad_embeddings, void* grad_offsets,
                                          void* stream) {
    if (grad_embeddings == nullptr) ASH_FAIL("accumulate: null grad_embeddings");
    return backward_forward(a, z, grad_embeddings, grad_offsets, stream, false);
}

int ash_query_backward_backward(const ash_query_args* a,
                                const void* grad_grad_offsets, const void* z,
                                void* grad_z, void* grad_embeddings,
                                void* stream) {
    return backward_backward(a, grad_grad_offsets, z, grad_z, grad_embeddings, stream, true);
}

int ash_query_backward_backward_accumulate(const ash_query_args* a,
                                           const void* grad_grad_offsets, const void* z,
                                           void* grad_z, void* grad_embeddings,
                                           void* stream) {
    if (grad_embeddings == nullptr) ASH_FAIL("accumulate: null grad_embeddings");
    return backward_backward(a, grad_grad_offsets, z, grad_z, grad_embeddings, stream, false);
}

namespace {

int convolution_forward(const void* inputs, const void* weights,
                        const uint8_t* masks, const int64_t* grid_indices,
                        const int64_t* cell_indices,
                        const int64_t* lut_grid_nb2grid_idx,
                        const int64_t* lut_cell_nb2cell_idx,
                        const int64_t* lut_cell_nb2grid_nb, void* outputs,
                        int64_t num_grids, int64_t num_embeddings,
                        int64_t cells_per_grid, int64_t embedding_dim,
                        int64_t num_cell_nbs, int64_t num_grid_nbs,
                        int32_t dtype, uint8_t* listed, void* stream) {
    if (dtype != ASH_F32 && dtype != ASH_F64) ASH_FAIL("unknown dtype");
    if (num_grids < 0 || num_embeddings < 1 || cells_per_grid < 1 ||
        embedding_dim < 1 || num_cell_nbs < 1 || num_grid_nbs < 1) {
        ASH_FAIL("convolution_forward: bad sizes");
    }
    if (inputs == nullptr || weights == nullptr || outputs == nullptr ||
        lut_grid_nb2grid_idx == nullptr || lut_cell_nb2cell_idx == nullptr ||
        lut_cell_nb2grid_nb == nullptr) {
        ASH_FAIL("null pointer in convolution_forward");
    }
    if (num_grids > 0 && (masks == nullptr || grid_indices == nullptr ||
                          cell_indices == nullptr)) {
        ASH_FAIL("null pointer in convolution_forward");
    }
    PointerGuard guard;
    ASH_HIP(guard.enter_for(inputs));
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t scalar = dtype == ASH_F32 ? 4 : 8;
    ConvDev a;
    a.in = inputs;
    a.w = weights;
    a.masks = masks;
    a.grid_indices = grid_indices;
    a.cell_indices = cell_indices;
    a.lut_g = lut_grid_nb2grid_idx;
    a.lut_c2c = lut_cell_nb2cell_idx;
    a.lut_c2g = lut_cell_nb2grid_nb;
    a.out = outputs;
    a.n_grids = num_grids;
    a.B = num_embeddings;
    a.M = cells_per_grid;
    a.E = embedding_dim;
    a.K = num_cell_nbs;
    a.GN = num_grid_nbs;
    a.owns = 0;
    // Rows of blocks that are not listed stay zero (at::zeros_like,
    // grid.cu:1010).  With a scratch byte per block and the tile kernel, which
    // writes every cell of the blocks it is given, only those rows are cleared.
    const int64_t block_bytes = cells_per_grid * embedding_dim * scalar;
    const bool tile = num_grids > 0 && embedding_dim <= 16 && num_cell_nbs >= kTileMinTaps &&
                      (dtype == ASH_F32 ? launch_convolution_tile<float>(a, s, true)
                                        : launch_convolution_tile<double>(a, s, true)) == 0;
    if (listed != nullptr && tile && block_bytes % 16 == 0 &&
        reinterpret_cast<uintptr_t>(outputs) % 16 == 0) {
        if (zero_fill(listed, num_embeddings, s)) return 1;
        mark_listed_kernel<<<static_cast<unsigned>((num_grids + kBlock - 1) / kBlock), kBlock, 0,
                             s>>>(grid_indices, num_grids, num_embeddings, listed);
        ASH_LAUNCH_CHECK();
        const int64_t g = num_embeddings < 256 * 32 ? num_embeddings : 256 * 32;
        zero_unlisted_kernel<<<static_cast<unsigned>(g), kBlock, 0, s>>>(
                static_cast<uint4*>(outputs), listed, num_embeddings, block_bytes / 16);
        ASH_LAUNCH_CHECK();
        a.owns = 1;
    } else if (zero_fill(outputs, num_embeddings * block_bytes, s)) {
        return 1;
    }
    if (num_grids == 0) return 0;
    if (embedding_dim <= 16) {
        return dtype == ASH_F32 ? launch_convolution_cells<float>(a, s)
                                : launch_convolution_cells<double>(a, s);
    }
    const int64_t threads = num_grids * cells_per_grid * embedding_dim;
    const int64_t blocks = (threads + kBlock - 1) / kBlock;
    if (blocks > 0x7FFFFFFFll) ASH_FAIL("convolution_forward: too many cells in one call");
    if (dtype == ASH_F32) {
        convolution_forward_kernel<float><<<static_cast<unsigned>(blocks), kBlock, 0, s>>>(a);
    } else {
        convolution_forward_kernel<double><<<static_cast<unsigned>(blocks), kBlock, 0, s>>>(a);
    }
    ASH_LAUNCH_CHECK();
    return 0;
}

}  // namespace

int ash_convolution_forward(const void* inputs, const void* weights,
                            const uint8_t* masks, const int64_t* grid_indices,
                            const int64_t* cell_indices,
                            const int64_t* lut_grid_nb2grid_idx,
                            const int64_t* lut_cell_nb2cell_idx,
                            const int64_t* lut_cell_nb2grid_nb, void* outputs,
                            int64_t num_grids, int64_t num_embeddings,
                            int64_t cells_per_grid, int64_t embedding_dim,
                            int64_t num_cell_nbs, int64_t num_grid_nbs,
                            int32_t dtype, void* stream) {
    return convolution_forward(inputs, weights, masks, grid_indices, cell_indices,
                               lut_grid_nb2grid_idx, lut_cell_nb2cell_idx, lut_cell_nb2grid_nb,
                               outputs, num_grids, num_embeddings, cells_per_grid, embedding_dim,
                               num_cell_nbs, num_grid_nbs, dtype, nullptr, stream);
}

int ash_convolution_forward_listed(const void* inputs, const void* weights,
                                   const uint8_t* masks, const int64_t* grid_indices,
                                   const int64_t* cell_indices,
                                   const int64_t* lut_grid_nb2grid_idx,
                                   const int64_t* lut_cell_nb2cell_idx,
                                   const int64_t* lut_cell_nb2grid_nb, void* outputs,
                                   int64_t num_grids, int64_t num_embeddings,
                                   int64_t cells_per_grid, int64_t embedding_dim,
                                   int64_t num_cell_nbs, int64_t num_grid_nbs,
                                   int32_t dtype, uint8_t* listed, void* stream) {
    if (listed == nullptr) ASH_FAIL("convolution_forward_listed: null scratch");
    return convolution_forward(inputs, weights, masks, grid_indices, cell_indices,
                               lut_grid_nb2grid_idx, lut_cell_nb2cell_idx, lut_cell_nb2grid_nb,
                               outputs, num_grids, num_embeddings, cells_per_grid, embedding_dim,
                               num_cell_nbs, num_grid_nbs, dtype, listed, stream);
}

}  // extern "C"
