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

// The update of cell t of the listing (block t / m, cell t % m).
__device__ __forceinline__ void integrate_cell(const IntegrateArgs& a, int64_t t) {
    const int64_t blk = t / a.m;
    const int cell = static_cast<int>(t - blk * a.m);
    const int64_t row = a.grid_idx[blk];
    if (row < 0 || row >= a.rows) return;
    const int c[3] = {cell % a.g, (cell / a.g) % a.g, cell / (a.g * a.g)};
    float p[3];
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        const int ic = a.grid_xyz[blk * 3 + d] * a.g + c[d];
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
    float rgb[3] = {0.f, 0.f, 0.f};
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
                rgb[0] = a.color[pix * 3 + 0];
                rgb[1] = a.color[pix * 3 + 1];
                rgb[2] = a.color[pix * 3 + 2];
            }
        }
    }
    float sdf = __fsub_rn(reading, d);
    const bool ok = inside && reading > 0.f && reading < a.depth_max && sdf >= -a.trunc;
    if (sdf >= a.trunc) sdf = a.trunc;
    const float weight = ok ? 1.f : 0.f;

    float* e = a.emb + (row * a.m + cell) * a.e;
    const float w_sum = e[a.e - 1];
    const float w_new = __fadd_rn(w_sum, weight);
    const float denom = __fadd_rn(w_new, 1e-6f);
    e[0] = __fdiv_rn(__fadd_rn(__fmul_rn(e[0], w_sum), __fmul_rn(sdf, weight)), denom);
    if (a.color != nullptr) {
#pragma unroll
        for (int q = 0; q < 3; ++q) {
            e[1 + q] = __fdiv_rn(
                    __fadd_rn(__fmul_rn(e[1 + q], w_sum), __fmul_rn(rgb[q], weight)), denom);
        }
    }
    e[a.e - 1] = w_new;
}

__global__ __launch_bounds__(kBlock) void integrate_depth_kernel(IntegrateArgs a) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (t < a.n * a.m) integrate_cell(a, t);
}

// The same over a listing whose length is on the device (`count`, at most
// a.n): a fixed grid strides over count * m cells, so no host value depends on
// the activation that made the listing.
__global__ __launch_bounds__(kBlock) void integrate_depth_counted_kernel(
        IntegrateArgs a, const int32_t* __restrict__ count) {
    int64_t blocks = *count;
    if (blocks > a.n) blocks = a.n;
    const int64_t cells = blocks * a.m;
    for (int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; t < cells;
         t += static_cast<int64_t>(gridDim.x) * kBlock) {
        integrate_cell(a, t);
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
    integrate_depth_counted_kernel<<<static_cast<unsigned>(blocks), kBlock, 0,
                                     static_cast<hipStream_t>(stream)>>>(
            a, map->d.ctr + kCtrTouched);
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
    integrate_depth_kernel<<<static_cast<unsigned>(blocks), kBlock, 0,
                             static_cast<hipStream_t>(stream)>>>(a);
    ASH_LAUNCH_CHECK();
    return 0;
}
