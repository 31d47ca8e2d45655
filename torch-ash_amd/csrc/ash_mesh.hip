// Marching cubes over the active blocks of a sparse-dense grid
// (ash/src/grid.cu:606-946 of the reference).
//
// The reference keeps an int case and three int vertex ids for every cell of
// all num_embeddings rows, zeroes both arrays and counts the marked edges with
// a full-array reduction.  Here a cell keeps one byte (its case) and one
// 32-bit word: bits 0..2 say which of the cell's own +x/+y/+z edges carry a
// surface vertex, bits 3..31 the id of the first of them; the ids of a cell's
// edges are consecutive, so `first + popcount(lower flagged axes)` addresses
// any of them.  Only the rows that are listed are cleared, and all counters are
// updated once per workgroup.
//
//   classify: clear listed rows -> case per cell, flags on the owning cells of
//             crossed edges, triangle count -> count of flagged edges
//   extract : ids + positions of the vertices -> triangles
//
// A cell takes part when it and the seven cells at its other corners exist
// and weigh at least the threshold; its case has bit c set when corner c is
// below the iso value.  Vertex ids follow the order in which workgroups reach
// the shared counter, as in the reference, so two runs may number the same
// mesh differently.
#include "ash_dev.h"
#include "ash_mc_table.h"

#include "../../include/ash_hip.h"

namespace ash {
namespace {

constexpr int kBlock = 256;
constexpr int64_t kMaxVertices = int64_t{1} << 29;  // ids live in 29 bits

enum McCounter {
    kMcCtrTriangles = 0,
    kMcCtrVertices = 1,
    kMcCtrVertexCursor = 2,
    kMcCtrTriangleCursor = 3
};

struct McDev {
    const void* sdfs;
    const void* weights;
    const int64_t* grid_indices;
    const int32_t* grid_coords;   // [B, 3] by row
    const int64_t* lut_g;         // [B, 8]
    const int32_t* cell_coords;   // [M, 3]
    const int64_t* lut_c2c;       // [M, 8]
    const int64_t* lut_c2g;       // [M, 8]
    uint8_t* cases;               // [B * M]
    uint32_t* slots;              // [B * M]
    int32_t* counters;            // [4]
    float* positions;             // [V, 3]
    int32_t* triangles;           // [T, 3]
    int64_t n_grids, B, M;
    int64_t n_vertices, n_triangles;
    float iso, weight_thr;
    int g;
};

// Exclusive prefix of `mine` over the workgroup and, in `first`, the value the
// shared counter had before the workgroup's total was added to it.
__device__ __forceinline__ int block_reserve(int mine, int32_t* counter, int& first) {
    __shared__ int s_cnt[kBlock / 64];
    __shared__ int s_first;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    int incl = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d);
        if (lane >= d) incl += up;
    }
    if (lane == 63) s_cnt[wave] = incl;
    __syncthreads();
    if (threadIdx.x == 0) {
        int tot = 0;
#pragma unroll
        for (int q = 0; q < kBlock / 64; ++q) {
            const int v = s_cnt[q];
            s_cnt[q] = tot;
            tot += v;
        }
        s_first = tot ? atomicAdd(counter, tot) : 0;
    }
    __syncthreads();
    first = s_first;
    return s_cnt[wave] + incl - mine;
}

// Row and cell of the cell at corner `nb` (0..7) of cell (g, c); false when the
// block that would hold it is not in the table.
__device__ __forceinline__ bool corner_cell(const McDev& a, int64_t g, int64_t c, int nb,
                                            int64_t& gi, int64_t& ci) {
    if (nb == 0) {
        gi = g;
        ci = c;
        return true;
    }
    const int64_t gn = a.lut_c2g[c * 8 + nb];
    gi = (gn >= 0 && gn < 8) ? a.lut_g[g * 8 + gn] : -1;
    if (gi < 0 || gi >= a.B) return false;
    ci = a.lut_c2c[c * 8 + nb];
    return ci >= 0 && ci < a.M;
}

__device__ __forceinline__ int edge_low_corner(int e) {
    const int axis = e >> 2;
    const int j = e & 3;
    return (j & ((1 << axis) - 1)) | ((j >> axis) << (axis + 1));
}

__global__ __launch_bounds__(kBlock) void mc_clear_kernel(McDev a) {
    const int64_t item = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (item < 4 && blockIdx.x == 0) a.counters[item] = 0;
    if (item >= a.n_grids * a.M) return;
    const int64_t g = a.grid_indices[item / a.M];
    if (g < 0 || g >= a.B) return;
    const int64_t at = g * a.M + item % a.M;
    a.cases[at] = 0;
    a.slots[at] = 0u;
}

__global__ void mc_reset_cursors_kernel(int32_t* counters) {
    if (threadIdx.x == 0) {
        counters[kMcCtrVertexCursor] = 0;
        counters[kMcCtrTriangleCursor] = 0;
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void mc_classify_kernel(McDev a) {
    const int64_t item = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const T* sdfs = static_cast<const T*>(a.sdfs);
    const T* weights = static_cast<const T*>(a.weights);
    int ntri = 0;
    if (item < a.n_grids * a.M) {
        const int64_t g = a.grid_indices[item / a.M];
        const int64_t c = item % a.M;
        if (g >= 0 && g < a.B) {
            int64_t at[8];
            bool valid = true;
            int code = 0;
#pragma unroll
            for (int nb = 0; nb < 8; ++nb) {
                int64_t gi, ci;
                if (!valid || !corner_cell(a, g, c, nb, gi, ci)) {
                    valid = false;
                    continue;
                }
                at[nb] = gi * a.M + ci;
                if (weights[at[nb]] < static_cast<T>(a.weight_thr)) {
                    valid = false;
                    continue;
                }
                const T diff = sdfs[at[nb]] - static_cast<T>(a.iso);
                code |= (diff < T(0)) << nb;
            }
            if (valid && code != 0 && code != 255) {
                a.cases[at[0]] = static_cast<uint8_t>(code);
                ntri = kMcTriangleCount[code];
#pragma unroll
                for (int e = 0; e < 12; ++e) {
                    const int axis = e >> 2;
                    const int low = edge_low_corner(e);
                    if (((code >> low) ^ (code >> (low | (1 << axis)))) & 1) {
                        atomicOr(a.slots + at[low], 1u << axis);
                    }
                }
            }
        }
    }
    int first;
    block_reserve(ntri, a.counters + kMcCtrTriangles, first);
}

__global__ __launch_bounds__(kBlock) void mc_count_vertices_kernel(McDev a) {
    const int64_t item = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    int mine = 0;
    if (item < a.n_grids * a.M) {
        const int64_t g = a.grid_indices[item / a.M];
        if (g >= 0 && g < a.B) mine = __popc(a.slots[g * a.M + item % a.M] & 7u);
    }
    int first;
    block_reserve(mine, a.counters + kMcCtrVertices, first);
}

// Gives the flagged edges of every cell their ids and writes the vertices:
// the zero crossing of the field along the edge, linear between its two ends
// (ash/src/grid.cu:748-771).
template <typename T>
__global__ __launch_bounds__(kBlock) void mc_vertices_kernel(McDev a) {
    const int64_t item = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const T* sdfs = static_cast<const T*>(a.sdfs);
    int flags = 0;
    int64_t g = -1;
    int64_t c = 0;
    if (item < a.n_grids * a.M) {
        g = a.grid_indices[item / a.M];
        c = item % a.M;
        if (g >= 0 && g < a.B) flags = static_cast<int>(a.slots[g * a.M + c] & 7u);
    }
    const int mine = __popc(flags);
    int first;
    const int before = block_reserve(mine, a.counters + kMcCtrVertexCursor, first);
    if (mine == 0) return;
    int64_t out = static_cast<int64_t>(first) + before;
    a.slots[g * a.M + c] = static_cast<uint32_t>(flags) | (static_cast<uint32_t>(out) << 3);
    if (out + mine > a.n_vertices) return;  // never with the counts of classify
    const T self = sdfs[g * a.M + c] - static_cast<T>(a.iso);
    float base[3];
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        base[d] = static_cast<float>(a.grid_coords[g * 3 + d] * a.g + a.cell_coords[c * 3 + d]);
    }
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        if (!(flags & (1 << d))) continue;
        int64_t gi, ci;
        float ratio = 0.f;
        if (corner_cell(a, g, c, 1 << d, gi, ci)) {
            const T other = sdfs[gi * a.M + ci] - static_cast<T>(a.iso);
            ratio = static_cast<float>(self / (self - other));
        }
        float* p = a.positions + out * 3;
        p[0] = base[0] + (d == 0 ? ratio : 0.f);
        p[1] = base[1] + (d == 1 ? ratio : 0.f);
        p[2] = base[2] + (d == 2 ? ratio : 0.f);
        ++out;
    }
}

// Triangles of every cell with a case, as ids of the vertices on its edges
// (ash/src/grid.cu:796-842).  The table rows already have the orientation the
// reference writes: normals point from below the iso value to above it.
__global__ __launch_bounds__(kBlock) void mc_triangles_kernel(McDev a) {
    const int64_t item = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    int code = 0;
    int64_t g = -1;
    int64_t c = 0;
    if (item < a.n_grids * a.M) {
        g = a.grid_indices[item / a.M];
        c = item % a.M;
        if (g >= 0 && g < a.B) code = a.cases[g * a.M + c];
    }
    const int mine = kMcTriangleCount[code];
    int first;
    const int before = block_reserve(mine, a.counters + kMcCtrTriangleCursor, first);
    if (mine == 0) return;
    const int64_t out = static_cast<int64_t>(first) + before;
    if (out + mine > a.n_triangles) return;  // never with the counts of classify
    // vertex ids of the crossed edges, looked up once per edge
    int32_t vid[12];
#pragma unroll
    for (int e = 0; e < 12; ++e) {
        const int axis = e >> 2;
        const int low = edge_low_corner(e);
        vid[e] = -1;
        if (((code >> low) ^ (code >> (low | (1 << axis)))) & 1) {
            int64_t gi, ci;
            if (corner_cell(a, g, c, low, gi, ci)) {
                const uint32_t slot = a.slots[gi * a.M + ci];
                vid[e] = static_cast<int32_t>(slot >> 3) +
                         __popc(slot & ((1u << axis) - 1u));
            }
        }
    }
    const int8_t* row = kMcTriangles[code];
    for (int t = 0; t < mine; ++t) {
        int32_t* tri = a.triangles + (out + t) * 3;
#pragma unroll
        for (int v = 0; v < 3; ++v) {
            const int e = row[3 * t + v];
            int32_t id = -1;
#pragma unroll
            for (int q = 0; q < 12; ++q) {
                if (q == e) id = vid[q];
            }
            tri[v] = id;
        }
    }
}

int fill_common(McDev& a, const void* sdfs, const int64_t* grid_indices,
                const int64_t* lut_g, const int64_t* lut_c2c, const int64_t* lut_c2g,
                int64_t num_grids, int64_t num_embeddings, int64_t cells_per_grid,
                float iso_value, int32_t dtype, uint8_t* cases, uint32_t* slots,
                int32_t* counters) {
    if (dtype != ASH_F32 && dtype != ASH_F64) ASH_FAIL("unknown dtype");
    if (num_grids < 0 || num_embeddings < 1 || cells_per_grid < 1) {
        ASH_FAIL("marching_cubes: bad sizes");
    }
    if (counters == nullptr) ASH_FAIL("marching_cubes: null counters");
    if (num_grids > 0 &&
        (sdfs == nullptr || grid_indices == nullptr || lut_g == nullptr ||
         lut_c2c == nullptr || lut_c2g == nullptr || cases == nullptr || slots == nullptr)) {
        ASH_FAIL("null pointer in marching_cubes");
    }
    const int64_t blocks = (num_grids * cells_per_grid + kBlock - 1) / kBlock;
    if (blocks > 0x7FFFFFFFll) ASH_FAIL("marching_cubes: too many cells in one call");
    a.sdfs = sdfs;
    a.grid_indices = grid_indices;
    a.lut_g = lut_g;
    a.lut_c2c = lut_c2c;
    a.lut_c2g = lut_c2g;
    a.cases = cases;
    a.slots = slots;
    a.counters = counters;
    a.n_grids = num_grids;
    a.B = num_embeddings;
    a.M = cells_per_grid;
    a.iso = iso_value;
    return 0;
}

}  // namespace
}  // namespace ash

using namespace ash;

extern "C" {

int ash_marching_cubes_classify(const void* sdfs, const void* weights,
                                const int64_t* grid_indices,
                                const int64_t* lut_grid_nb2grid_idx,
                                const int64_t* lut_cell_nb2cell_idx,
                                const int64_t* lut_cell_nb2grid_nb, int64_t num_grids,
                                int64_t num_embeddings, int64_t cells_per_grid,
                                float iso_value, float weight_thr, int32_t dtype,
                                uint8_t* cases, uint32_t* edge_slots, int32_t* counters,
                                void* stream) {
    McDev a = {};
    if (fill_common(a, sdfs, grid_indices, lut_grid_nb2grid_idx, lut_cell_nb2cell_idx,
                    lut_cell_nb2grid_nb, num_grids, num_embeddings, cells_per_grid,
                    iso_value, dtype, cases, edge_slots, counters)) {
        return 1;
    }
    if (num_grids > 0 && weights == nullptr) ASH_FAIL("null pointer in marching_cubes");
    a.weights = weights;
    a.weight_thr = weight_thr;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t cells = num_grids * cells_per_grid;
    const unsigned blocks = static_cast<unsigned>((cells + kBlock - 1) / kBlock);
    mc_clear_kernel<<<blocks ? blocks : 1, kBlock, 0, s>>>(a);
    ASH_LAUNCH_CHECK();
    if (num_grids == 0) return 0;
    if (dtype == ASH_F32) {
        mc_classify_kernel<float><<<blocks, kBlock, 0, s>>>(a);
    } else {
        mc_classify_kernel<double><<<blocks, kBlock, 0, s>>>(a);
    }
    ASH_LAUNCH_CHECK();
    mc_count_vertices_kernel<<<blocks, kBlock, 0, s>>>(a);
    ASH_LAUNCH_CHECK();
    return 0;
}

int ash_marching_cubes_extract(const void* sdfs, const int64_t* grid_indices,
                               const int32_t* grid_coords_table,
                               const int64_t* lut_grid_nb2grid_idx,
                               const int32_t* cell_coords_table,
                               const int64_t* lut_cell_nb2cell_idx,
                               const int64_t* lut_cell_nb2grid_nb, int64_t num_grids,
                               int64_t num_embeddings, int64_t cells_per_grid, int grid_dim,
                               float iso_value, int32_t dtype, const uint8_t* cases,
                               uint32_t* edge_slots, int32_t* counters, int64_t n_vertices,
                               int64_t n_triangles, float* positions, int32_t* triangles,
                               void* stream) {
    McDev a = {};
    if (fill_common(a, sdfs, grid_indices, lut_grid_nb2grid_idx, lut_cell_nb2cell_idx,
                    lut_cell_nb2grid_nb, num_grids, num_embeddings, cells_per_grid,
                    iso_value, dtype, const_cast<uint8_t*>(cases), edge_slots, counters)) {
        return 1;
    }
    if (grid_dim < 1) ASH_FAIL("marching_cubes: bad sizes");
    if (n_vertices < 0 || n_triangles < 0) ASH_FAIL("marching_cubes: negative counts");
    if (n_vertices >= kMaxVertices) ASH_FAIL("marching_cubes: more than 2^29 vertices");
    if (num_grids == 0 || (n_vertices == 0 && n_triangles == 0)) return 0;
    if (grid_coords_table == nullptr || cell_coords_table == nullptr ||
        (n_vertices > 0 && positions == nullptr) ||
        (n_triangles > 0 && triangles == nullptr)) {
        ASH_FAIL("null pointer in marching_cubes");
    }
    a.grid_coords = grid_coords_table;
    a.cell_coords = cell_coords_table;
    a.positions = positions;
    a.triangles = triangles;
    a.n_vertices = n_vertices;
    a.n_triangles = n_triangles;
    a.g = grid_dim;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t cells = num_grids * cells_per_grid;
    const unsigned blocks = static_cast<unsigned>((cells + kBlock - 1) / kBlock);
    mc_reset_cursors_kernel<<<1, 64, 0, s>>>(counters);
    ASH_LAUNCH_CHECK();
    if (dtype == ASH_F32) {
        mc_vertices_kernel<float><<<blocks, kBlock, 0, s>>>(a);
    } else {
        mc_vertices_kernel<double><<<blocks, kBlock, 0, s>>>(a);
    }
    ASH_LAUNCH_CHECK();
    if (n_triangles > 0) {
        mc_triangles_kernel<<<blocks, kBlock, 0, s>>>(a);
        ASH_LAUNCH_CHECK();
    }
    return 0;
}

}  // extern "C"
