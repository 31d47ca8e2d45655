// Depth integration into a sparse-dense grid: the per-frame update of a TSDF
// fusion loop (demo/rgbd_fusion.py:76-110,216-254 of the reference) as one
// kernel.  The reference gathers embeddings[grid_indices, cell_indices],
// projects every cell with two small matrix products, reads depth / colour by
// advanced indexing, forms the running weighted mean and scatters the rows
// back -- about thirty launches and several (blocks x 512)-row temporaries.
// Here one thread owns one cell of one touched block and updates its embedding
// row in place.
//
// Row layout, as in the reference demo: channel 0 = signed distance, last
// channel = accumulated weight, channels 1..3 = colour when a colour image is
// given.  The arithmetic of the update is evaluated operation by operation in
// fp32 (no fused multiply-add), i.e. exactly like the elementwise torch
// expressions; the projection uses fused multiply-adds where torch calls a
// matrix product, whose rounding is not specified either.
#include "ash_table.h"

#include "../../include/ash_hip.h"

namespace ash {
namespace {

constexpr int kBlock = 256;
constexpr int kFlaggedGroups = 8192;    // workgroups of the integration that goes by flags

struct IntegrateArgs {
    float* emb;                // [B, M, E]
    const int64_t* grid_idx;   // [n] rows of emb
    const int32_t* grid_xyz;   // [n, 3] block coordinates
    const float* intrinsic;    // 3x3 row-major (device)
    const float* extrinsic;    // 4x4 row-major world -> camera (device)
    const float* depth;        // [H, W]
    const float* color;        // [H, W, 3] or nullptr
    int64_t n;
    int64_t rows;              // B
    int g, m, e, h, w;
    float cell_size;
    float origin[3];
    int has_origin;
    float trunc, depth_max;
};

// What the frame says about one cell: the truncated signed distance along the
// viewing ray, the weight of the observation (0 or 1) and the colour.
struct CellObservation {
    float sdf, weight;
    float rgb[3];
};

// Projects cell `cell` of the block at bx, by, bz into the frame.  G: cells
// per block edge when known at compile time (shifts instead of divisions),
// else 0 and a.g is used.
template <int G>
__device__ __forceinline__ CellObservation observe_cell(const IntegrateArgs& a, int cell, int bx,
                                                        int by, int bz) {
    const int g = G > 0 ? G : a.g;
    const int c[3] = {cell % g, (cell / g) % g, cell / (g * g)};
    const int b[3] = {bx, by, bz};
    float p[3];
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        const int ic = b[d] * g + c[d];
        p[d] = __fmul_rn(static_cast<float>(ic), a.cell_size);
        if (a.has_origin) p[d] = __fadd_rn(p[d], a.origin[d]);
    }
    const float* T = a.extrinsic;
    const float* K = a.intrinsic;
    float cam[3];
#pragma unroll
    for (int r = 0; r < 3; ++r) {
        cam[r] = fmaf(p[2], T[r * 4 + 2], fmaf(p[1], T[r * 4 + 1], p[0] * T[r * 4 + 0])) +
                 T[r * 4 + 3];
    }
    float uvd[3];
#pragma unroll
    for (int r = 0; r < 3; ++r) {
        uvd[r] = fmaf(cam[2], K[r * 3 + 2], fmaf(cam[1], K[r * 3 + 1], cam[0] * K[r * 3 + 0]));
    }
    const float d = uvd[2];
    float reading = 0.f;
    CellObservation o = {0.f, 0.f, {0.f, 0.f, 0.f}};
    bool inside = false;
    if (d > 0.f) {
        const float uf = rintf(__fdiv_rn(uvd[0], d));
        const float vf = rintf(__fdiv_rn(uvd[1], d));
        inside = uf >= 0.f && vf >= 0.f && uf < static_cast<float>(a.w) &&
                 vf < static_cast<float>(a.h);
        if (inside) {
            const int64_t pix = static_cast<int64_t>(vf) * a.w + static_cast<int64_t>(uf);
            reading = a.depth[pix];
            if (a.color != nullptr) {
                o.rgb[0] = a.color[pix * 3 + 0];
                o.rgb[1] = a.color[pix * 3 + 1];
                o.rgb[2] = a.color[pix * 3 + 2];
            }
        }
    }
    o.sdf = __fsub_rn(reading, d);
    const bool ok = inside && reading > 0.f && reading < a.depth_max && o.sdf >= -a.trunc;
    if (o.sdf >= a.trunc) o.sdf = a.trunc;
    o.weight = ok ? 1.f : 0.f;
    return o;
}

// A row of distance and weight after the observation: the running weighted
// mean of demo/rgbd_fusion.py:232-254, operation by operation.
__device__ __forceinline__ float2 folded(const float2 old, const CellObservation& o) {
    const float w_new = __fadd_rn(old.y, o.weight);
    const float denom = __fadd_rn(w_new, 1e-6f);
    float2 out;
    out.x = __fdiv_rn(__fadd_rn(__fmul_rn(old.x, old.y), __fmul_rn(o.sdf, o.weight)), denom);
    out.y = w_new;
    return out;
}

// The same for a row of distance, colour and weight (five channels, 20 bytes,
// 4-byte aligned: moved as 16 + 4 bytes); without a colour image the three
// colour channels keep what they hold.
struct alignas(4) Row5 {
    float v[5];
};

__device__ __forceinline__ Row5 folded(const Row5& old, const CellObservation& o, bool colour) {
    const float w_sum = old.v[4];
    const float w_new = __fadd_rn(w_sum, o.weight);
    const float denom = __fadd_rn(w_new, 1e-6f);
    Row5 out = old;
    out.v[0] = __fdiv_rn(__fadd_rn(__fmul_rn(old.v[0], w_sum), __fmul_rn(o.sdf, o.weight)), denom);
    if (colour) {
#pragma unroll
        for (int q = 0; q < 3; ++q) {
            out.v[1 + q] = __fdiv_rn(
                    __fadd_rn(__fmul_rn(old.v[1 + q], w_sum), __fmul_rn(o.rgb[q], o.weight)), denom);
        }
    }
    out.v[4] = w_new;
    return out;
}

// The update of cell `cell` of the block stored in row `row` of the
// embeddings, whose block coordinates are bx, by, bz.  E: channels per row
// when known at compile time (2: one 8-byte access per row; 5: 16 + 4 bytes),
// else 0 and a.e is used.  Either way the arithmetic of the update is the same sequence of fp32
// operations.
template <int G, int E>
__device__ __forceinline__ void integrate_cell_at(const IntegrateArgs& a, int64_t row, int cell,
                                                  int bx, int by, int bz) {
    const int ne = E > 0 ? E : a.e;
    const CellObservation o = observe_cell<G>(a, cell, bx, by, bz);
    float* e = a.emb + (row * (G > 0 ? G * G * G : a.m) + cell) * ne;
    if constexpr (E == 2) {
        float2* e2 = reinterpret_cast<float2*>(e);
        *e2 = folded(*e2, o);
    } else if constexpr (E == 5) {
        Row5* e5 = reinterpret_cast<Row5*>(e);
        *e5 = folded(*e5, o, a.color != nullptr);
    } else {
        const float w_sum = e[ne - 1];
        const float w_new = __fadd_rn(w_sum, o.weight);
        const float denom = __fadd_rn(w_new, 1e-6f);
        e[0] = __fdiv_rn(__fadd_rn(__fmul_rn(e[0], w_sum), __fmul_rn(o.sdf, o.weight)), denom);
        if (a.color != nullptr) {
#pragma unroll
            for (int q = 0; q < 3; ++q) {
                e[1 + q] = __fdiv_rn(
                        __fadd_rn(__fmul_rn(e[1 + q], w_sum), __fmul_rn(o.rgb[q], o.weight)), denom);
            }
        }
        e[ne - 1] = w_new;
    }
}

// The update of cell t of the listing (block t / m, cell t % m).
template <int G, int E>
__device__ __forceinline__ void integrate_cell(const IntegrateArgs& a, int64_t t) {
    const int m = G > 0 ? G * G * G : a.m;
    const int64_t blk = t / m;
    const int cell = static_cast<int>(t - blk * m);
    const int64_t row = a.grid_idx[blk];
    if (row < 0 || row >= a.rows) return;
    integrate_cell_at<G, E>(a, row, cell, a.grid_xyz[blk * 3 + 0], a.grid_xyz[blk * 3 + 1],
                            a.grid_xyz[blk * 3 + 2]);
}

template <int G, int E>
__global__ __launch_bounds__(kBlock) void integrate_depth_kernel(IntegrateArgs a) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (t < a.n * a.m) integrate_cell<G, E>(a, t);
}

// The same over a listing whose length is on the device (`count`, at most
// a.n): a fixed grid strides over count * m cells, so no host value depends on
// the activation that made the listing.
template <int G, int E>
__global__ __launch_bounds__(kBlock) void integrate_depth_counted_kernel(
        IntegrateArgs a, const int32_t* __restrict__ count) {
    int64_t blocks = *count;
    if (blocks > a.n) blocks = a.n;
    const int64_t cells = blocks * a.m;
    for (int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; t < cells;
         t += static_cast<int64_t>(gridDim.x) * kBlock) {
        integrate_cell<G, E>(a, t);
    }
}

// The same over the rows an activation has flagged, without a listing:
// workgroup w looks at the flags of rows w, w + W, w + 2 W, ... (rows in use
// are the low ones as a rule, so every workgroup gets its share of them),
// kBlock flags per round, lists the flagged ones in LDS, takes the flags down
// and updates the cells of the listed blocks, whose coordinates stand in
// coords[row].  a.grid_idx is not used; a.n is the number of rows.
template <int G, int E>
__global__ __launch_bounds__(kBlock) void integrate_depth_flagged_kernel(
        IntegrateArgs a, uint8_t* __restrict__ touched) {
    __shared__ int32_t s_rows[kBlock * 4];   // row and block coordinates of the flagged ones
    __shared__ int s_n;
    const int m = G > 0 ? G * G * G : a.m;
    const int64_t stride = gridDim.x;
    for (int64_t first = blockIdx.x; first < a.n; first += stride * kBlock) {
        if (threadIdx.x == 0) s_n = 0;
        __syncthreads();
        const int64_t row = first + static_cast<int64_t>(threadIdx.x) * stride;
        if (row < a.n) {
            // the coordinates are asked for with the flag, not after it
            const uint8_t flag = touched[row];
            const int32_t cx = a.grid_xyz[row * 3 + 0];
            const int32_t cy = a.grid_xyz[row * 3 + 1];
            const int32_t cz = a.grid_xyz[row * 3 + 2];
            if (flag != 0) touched[row] = 0;
            if (flag != 0 && row < a.rows) {   // (a flagged row without embeddings is let go)
                const int at = atomicAdd(&s_n, 1);
                s_rows[at * 4 + 0] = static_cast<int32_t>(row);
                s_rows[at * 4 + 1] = cx;
                s_rows[at * 4 + 2] = cy;
                s_rows[at * 4 + 3] = cz;
            }
        }
        __syncthreads();
        const int listed = s_n;
        for (int j = 0; j < listed; ++j) {
            const int32_t r = s_rows[j * 4 + 0];
            const int bx = s_rows[j * 4 + 1];
            const int by = s_rows[j * 4 + 2];
            const int bz = s_rows[j * 4 + 3];
            if constexpr (E == 2) {
                // two cells per thread and turn, their rows asked for before
                // either projection: one wait for memory instead of two
                float2* rows = reinterpret_cast<float2*>(a.emb) + static_cast<int64_t>(r) * m;
                for (int cell = threadIdx.x; cell < m; cell += 2 * kBlock) {
                    const int other = cell + kBlock;
                    const bool two = other < m;
                    const float2 old0 = rows[cell];
                    const float2 old1 = two ? rows[other] : make_float2(0.f, 0.f);
                    const CellObservation o0 = observe_cell<G>(a, cell, bx, by, bz);
                    const CellObservation o1 = observe_cell<G>(a, two ? other : cell, bx, by, bz);
                    rows[cell] = folded(old0, o0);
                    if (two) rows[other] = folded(old1, o1);
                }
            } else if constexpr (E == 5) {
                Row5* rows = reinterpret_cast<Row5*>(a.emb) + static_cast<int64_t>(r) * m;
                const bool colour = a.color != nullptr;
                for (int cell = threadIdx.x; cell < m; cell += 2 * kBlock) {
                    const int other = cell + kBlock;
                    const bool two = other < m;
                    const Row5 old0 = rows[cell];
                    const Row5 old1 = rows[two ? other : cell];
                    const CellObservation o0 = observe_cell<G>(a, cell, bx, by, bz);
                    const CellObservation o1 = observe_cell<G>(a, two ? other : cell, bx, by, bz);
                    rows[cell] = folded(old0, o0, colour);
                    if (two) rows[other] = folded(old1, o1, colour);
                }
            } else {
                for (int cell = threadIdx.x; cell < m; cell += kBlock) {
                    integrate_cell_at<G, E>(a, r, cell, bx, by, bz);
                }
            }
        }
        __syncthreads();   // s_rows and s_n are rewritten by the next round
    }
}

}  // namespace
}  // namespace ash

using namespace ash;

namespace {

int fill_integrate_args(IntegrateArgs& a, float* embeddings, int64_t num_embeddings,
                        int grid_dim, int embedding_dim, const int64_t* grid_indices,
                        const int32_t* grid_coords, int64_t n_blocks, float cell_size,
                        const float* origin, const float* intrinsic, const float* extrinsic,
                        const float* depth, const float* color, int height, int width,
                        float trunc, float depth_max) {
    if (embeddings == nullptr || grid_indices == nullptr || grid_coords == nullptr ||
        intrinsic == nullptr || extrinsic == nullptr || depth == nullptr) {
        ASH_FAIL("null pointer in depth integration");
    }
    if (grid_dim < 1 || grid_dim > 64) ASH_FAIL("grid_dim must be in 1..64");
    if (embedding_dim < 2) ASH_FAIL("rows need a distance and a weight channel");
    if (color != nullptr && embedding_dim < 5) {
        ASH_FAIL("rows need five channels to integrate colour");
    }
    if (height < 1 || width < 1) ASH_FAIL("empty depth image");
    if (num_embeddings < 1) ASH_FAIL("empty embedding table");
    a.emb = embeddings;
    a.grid_idx = grid_indices;
    a.grid_xyz = grid_coords;
    a.intrinsic = intrinsic;
    a.extrinsic = extrinsic;
    a.depth = depth;
    a.color = color;
    a.n = n_blocks;
    a.rows = num_embeddings;
    a.g = grid_dim;
    a.m = grid_dim * grid_dim * grid_dim;
    a.e = embedding_dim;
    a.h = height;
    a.w = width;
    a.cell_size = cell_size;
    a.has_origin = origin != nullptr;
    for (int d = 0; d < 3; ++d) a.origin[d] = origin ? origin[d] : 0.f;
    a.trunc = trunc;
    a.depth_max = depth_max;
    if (n_blocks * a.m > (int64_t{1} << 40)) ASH_FAIL("too many cells in one call");
    return 0;
}

}  // namespace

extern "C" int ash_grid_integrate_depth_touched(
        ash_map_t* map, float* embeddings, int64_t num_embeddings, int grid_dim,
        int embedding_dim, const int64_t* grid_indices, const int32_t* grid_coords,
        float cell_size, const float* origin, const float* intrinsic, const float* extrinsic,
        const float* depth, const float* color, int height, int width, float trunc,
        float depth_max, void* stream) {
    if (map == nullptr) ASH_FAIL("null map handle");
    IntegrateArgs a;
    if (fill_integrate_args(a, embeddings, num_embeddings, grid_dim, embedding_dim, grid_indices,
                            grid_coords, map->capacity, cell_size, origin, intrinsic, extrinsic,
                            depth, color, height, width, trunc, depth_max)) {
        return 1;
    }
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    // enough workgroups to fill the device; they stride over the listing
    int64_t blocks = (map->capacity * a.m + kBlock - 1) / kBlock;
    if (blocks > 256 * 16) blocks = 256 * 16;
    if (a.g == 8 && a.e == 2) {
        integrate_depth_counted_kernel<8, 2><<<static_cast<unsigned>(blocks), kBlock, 0,
                                               static_cast<hipStream_t>(stream)>>>(
                a, map->d.ctr + kCtrTouched);
    } else if (a.g == 8 && a.e == 5) {
        integrate_depth_counted_kernel<8, 5><<<static_cast<unsigned>(blocks), kBlock, 0,
                                               static_cast<hipStream_t>(stream)>>>(
                a, map->d.ctr + kCtrTouched);
    } else {
        integrate_depth_counted_kernel<0, 0><<<static_cast<unsigned>(blocks), kBlock, 0,
                                               static_cast<hipStream_t>(stream)>>>(
                a, map->d.ctr + kCtrTouched);
    }
    ASH_LAUNCH_CHECK();
    return 0;
}

extern "C" int ash_grid_integrate_depth_flagged(
        ash_map_t* map, float* embeddings, int64_t num_embeddings, int grid_dim,
        int embedding_dim, uint8_t* touched, const int32_t* coords, float cell_size,
        const float* origin, const float* intrinsic, const float* extrinsic,
        const float* depth, const float* color, int height, int width, float trunc,
        float depth_max, void* stream) {
    if (map == nullptr) ASH_FAIL("null map handle");
    if (touched == nullptr) ASH_FAIL("null pointer in depth integration");
    IntegrateArgs a;
    // (the listing argument is not used by this variant: the rows are their own
    // numbers and `coords` is indexed by row)
    if (fill_integrate_args(a, embeddings, num_embeddings, grid_dim, embedding_dim,
                            reinterpret_cast<const int64_t*>(touched), coords, map->capacity,
                            cell_size, origin, intrinsic, extrinsic, depth, color, height, width,
                            trunc, depth_max)) {
        return 1;
    }
    a.grid_idx = nullptr;
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    // rows are dealt out round robin: enough workgroups to fill the device,
    // few enough that each looks at its flags in one round as a rule
    int64_t groups = map->capacity < kFlaggedGroups ? map->capacity : kFlaggedGroups;
    if (groups < 1) groups = 1;
    if (a.g == 8 && a.e == 2) {
        integrate_depth_flagged_kernel<8, 2><<<static_cast<unsigned>(groups), kBlock, 0,
                                               static_cast<hipStream_t>(stream)>>>(a, touched);
    } else if (a.g == 8 && a.e == 5) {
        integrate_depth_flagged_kernel<8, 5><<<static_cast<unsigned>(groups), kBlock, 0,
                                               static_cast<hipStream_t>(stream)>>>(a, touched);
    } else {
        integrate_depth_flagged_kernel<0, 0><<<static_cast<unsigned>(groups), kBlock, 0,
                                               static_cast<hipStream_t>(stream)>>>(a, touched);
    }
    ASH_LAUNCH_CHECK();
    return 0;
}

extern "C" int ash_grid_integrate_depth(
        float* embeddings, int64_t num_embeddings, int grid_dim, int embedding_dim,
        const int64_t* grid_indices, const int32_t* grid_coords, int64_t n_blocks,
        float cell_size, const float* origin, const float* intrinsic,
        const float* extrinsic, const float* depth, const float* color, int height,
        int width, float trunc, float depth_max, void* stream) {
    if (n_blocks < 0) ASH_FAIL("negative block count");
    if (n_blocks == 0) return 0;
    IntegrateArgs a;
    if (fill_integrate_args(a, embeddings, num_embeddings, grid_dim, embedding_dim, grid_indices,
                            grid_coords, n_blocks, cell_size, origin, intrinsic, extrinsic, depth,
                            color, height, width, trunc, depth_max)) {
        return 1;
    }
    PointerGuard guard;
    ASH_HIP(guard.enter_for(embeddings));
    const int64_t threads = n_blocks * a.m;
    const int64_t blocks = (threads + kBlock - 1) / kBlock;
    if (blocks > 0x7FFFFFFFll) ASH_FAIL("too many cells in one call");
    if (a.g == 8 && a.e == 2) {
        integrate_depth_kernel<8, 2><<<static_cast<unsigned>(blocks), kBlock, 0,
                                       static_cast<hipStream_t>(stream)>>>(a);
    } else if (a.g == 8 && a.e == 5) {
        integrate_depth_kernel<8, 5><<<static_cast<unsigned>(blocks), kBlock, 0,
                                       static_cast<hipStream_t>(stream)>>>(a);
    } else {
        integrate_depth_kernel<0, 0><<<static_cast<unsigned>(blocks), kBlock, 0,
                                       static_cast<hipStream_t>(stream)>>>(a);
    }
    ASH_LAUNCH_CHECK();
    return 0;
}
