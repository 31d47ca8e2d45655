// Marching cubes over the active blocks of a sparse-dense grid
// (ash/src/grid.cu:606-946 of the reference).
//
// The reference keeps an int case and three int vertex ids for every cell of
// all num_embeddings rows, zeroes both arrays, counts the marked edges with a
// full-array reduction and takes one atomic on a single counter per vertex and
// per triangle.  Here a cell keeps one byte (its case) and one 32-bit word:
// bits 0..2 say which of the cell's own +x/+y/+z edges carry a surface vertex,
// bits 3..31 the id of the first of them; the ids of a cell's edges are
// consecutive, so `first + popcount(lower flagged axes)` addresses any of
// them.  Only the rows that are listed are cleared.  Updates of one address
// serialise in the memory system (several ns each, which at tens of thousands
// of workgroups is the run time of a pass), so no pass updates a shared
// counter: the cells of the listing are cut into chunks of 4096, a count pass
// stores per-chunk totals, one small workgroup turns them into running sums,
// and the output passes start from there -- which also makes the numbering of
// vertices and triangles the same on every run.
//
//   classify: clear listed rows
//             -> per block: stage "heavy enough" and "below iso" of the block's
//                (G+1)^3 corner cells in LDS, form the case of every cell from
//                there, flag the owning cells of crossed edges (byte stores)
//             -> per chunk: pack the flags, count flagged edges and triangles
//             -> running sums over the chunks, totals
//   extract : per chunk: compact the flagged cells in LDS, write ids +
//             positions -> same for the cells with a case: write triangles
//
// A cell takes part when it and the seven cells at its other corners exist
// and weigh at least the threshold; its case has bit c set when corner c is
// below the iso value.
#include "ash_table.h"
#include "ash_mc_table.h"

#include "../../include/ash_hip.h"

namespace ash {
namespace {

constexpr int kBlock = 256;
constexpr int kPerThread = 16;
constexpr int kChunk = kBlock * kPerThread;   // cells per reservation
constexpr int kMaxTileG = 16;                 // block edge handled by the LDS tile
constexpr int kMaxGrid = 65536;               // workgroups of a chunk launch: one per chunk up to here (8192: 5 % slower, 4096: 10 %)
constexpr int64_t kMaxVertices = int64_t{1} << 29;  // ids live in 29 bits

// Layout of the int32 workspace: totals, then per chunk of kChunk cells the
// number (after mc_scan_kernel: the running sum) of vertices and of triangles.
enum McWorkspace { kMcTriangles32 = 0, kMcVertices32 = 1, kMcStandard = 3, kMcHeader = 4 };

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
    int32_t* counters;            // workspace: totals, then per-chunk counts / running sums
    float* positions;             // [V, 3]
    int32_t* triangles;           // [T, 3]
    int64_t n_grids, B, M;
    int64_t n_vertices, n_triangles;
    float iso, weight_thr;
    int g;
};

// Exclusive prefix of `v` over the workgroup; `total` receives the sum.
__device__ __forceinline__ int block_exclusive(int v, int& total) {
    __shared__ int s_part[kBlock / 64];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    int incl = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d);
        if (lane >= d) incl += up;
    }
    __syncthreads();  // the previous use of s_part has been read
    if (lane == 63) s_part[wave] = incl;
    __syncthreads();
    int before = 0;
    int tot = 0;
#pragma unroll
    for (int q = 0; q < kBlock / 64; ++q) {
        const int p = s_part[q];
        if (q < wave) before += p;
        tot += p;
    }
    total = tot;
    return before + incl - v;
}

// v[j] = what the thread's group j contributes, two 16-bit counts packed into
// one int.  On return v[j] is the sum over all cells of the chunk that come
// before the group in cell order; the result is the chunk's total.
template <int GROUPS>
__device__ __forceinline__ int chunk_exclusive(int (&v)[GROUPS]) {
    __shared__ int s_part[kBlock / 64];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    int run = 0;
#pragma unroll
    for (int j = 0; j < GROUPS; ++j) {
        int incl = v[j];
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(incl, d);
            if (lane >= d) incl += up;
        }
        const int all = __shfl(incl, 63);
        v[j] = run + incl - v[j];
        run += all;
    }
    __syncthreads();  // the previous use of s_part has been read
    if (lane == 0) s_part[wave] = run;
    __syncthreads();
    int before = 0;
    int tot = 0;
#pragma unroll
    for (int q = 0; q < kBlock / 64; ++q) {
        const int p = s_part[q];
        if (q < wave) before += p;
        tot += p;
    }
#pragma unroll
    for (int j = 0; j < GROUPS; ++j) v[j] += before;
    return tot;
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

// The Python layer numbers cells x + G y + G^2 z and builds the two per-cell
// tables from that; layout_check_kernel compares the tables it is given with
// this layout and leaves the verdict in the workspace header (kMcStandard).
// The output kernels then work corners out instead of asking three tables in
// a row for each of them; any other tables are followed as before.
struct CellAt {
    int x, y, z;
};

__device__ __forceinline__ CellAt cell_at(int G, int c) {
    CellAt p;
    p.x = c % G;
    const int r = c / G;
    p.y = r % G;
    p.z = r / G;
    return p;
}

__device__ __forceinline__ bool corner_cell_standard(const McDev& a, int64_t g, const CellAt& p,
                                                     int nb, int64_t& gi, int64_t& ci) {
    const int G = a.g;
    const int tx = p.x + (nb & 1), ty = p.y + ((nb >> 1) & 1), tz = p.z + (nb >> 2);
    const int bx = tx >= G, by = ty >= G, bz = tz >= G;
    const int gn = bx | (by << 1) | (bz << 2);
    ci = (tx - bx * G) + G * ((ty - by * G) + G * (tz - bz * G));
    gi = gn == 0 ? g : a.lut_g[g * 8 + gn];
    return gi >= 0 && gi < a.B;
}

constexpr int kCheckThreads = 1024;

__global__ __launch_bounds__(kCheckThreads) void layout_check_kernel(McDev a) {
    __shared__ int s_bad;
    if (threadIdx.x == 0) s_bad = 0;
    __syncthreads();
    const int G = a.g;
    const int M = static_cast<int>(a.M);
    int bad = static_cast<int64_t>(G) * G * G != a.M;
    // no early way out of the loop: its loads are then all in flight together
#pragma unroll 4
    for (int t = threadIdx.x; t < (bad ? 0 : M * 8); t += kCheckThreads) {
        const int c = t >> 3;
        const int nb = t & 7;
        const CellAt p = cell_at(G, c);
        const int tx = p.x + (nb & 1), ty = p.y + ((nb >> 1) & 1), tz = p.z + (nb >> 2);
        const int bx = tx >= G, by = ty >= G, bz = tz >= G;
        const int64_t gn = bx | (by << 1) | (bz << 2);
        const int64_t ci = (tx - bx * G) + G * ((ty - by * G) + G * (tz - bz * G));
        bad |= a.lut_c2g[t] != gn || a.lut_c2c[t] != ci;
        if (nb == 0) {
            bad |= a.cell_coords[c * 3] != p.x || a.cell_coords[c * 3 + 1] != p.y ||
                   a.cell_coords[c * 3 + 2] != p.z;
        }
    }
    if (bad) s_bad = 1;
    __syncthreads();
    if (threadIdx.x == 0) a.counters[kMcStandard] = s_bad ? 0 : 1;
}

__device__ __forceinline__ int edge_low_corner(int e) {
    const int axis = e >> 2;
    const int j = e & 3;
    return (j & ((1 << axis) - 1)) | ((j >> axis) << (axis + 1));
}

__device__ __forceinline__ bool edge_crossed(int code, int e) {
    const int low = edge_low_corner(e);
    return ((code >> low) ^ (code >> (low | (1 << (e >> 2))))) & 1;
}

// During classify the three flags of a cell are the low bits of bytes 0..2 of
// its word, so that they can be set by plain byte stores from any workgroup.
__device__ __forceinline__ void flag_edge(const McDev& a, int64_t at, int axis) {
    reinterpret_cast<uint8_t*>(a.slots)[at * 4 + axis] = 1;
}

// The cells of chunk `chunk` (kChunk consecutive cells of the listing) that a
// thread owns: kPerThread / VEC groups of VEC consecutive cells.  A wavefront
// owns a contiguous quarter of the chunk and its lanes take the groups of that
// quarter round robin, so that a wavefront touches consecutive memory.  Calls
// f(j, offset of the group in the chunk, index of its first cell in the
// per-cell arrays) for groups that exist and whose block is a valid row.  With
// VEC > 1 the cells of a block must be a multiple of VEC.
template <int VEC>
__device__ __forceinline__ uint32_t own_group_offset(int j) {
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t lane = threadIdx.x & 63;
    return ((wave * (kPerThread / VEC) + j) * 64 + lane) * VEC;
}

template <int VEC, typename F>
__device__ __forceinline__ void for_own_groups(const McDev& a, int64_t chunk, F f) {
    const int64_t cells = a.n_grids * a.M;
    const int64_t base = chunk * kChunk;
    const int64_t blk0 = base / a.M;
    const uint32_t m = static_cast<uint32_t>(a.M);
    const uint32_t c0 = static_cast<uint32_t>(base - blk0 * a.M);
#pragma unroll
    for (int j = 0; j < kPerThread / VEC; ++j) {
        const uint32_t local = own_group_offset<VEC>(j);
        if (base + local >= cells) continue;
        const uint32_t o = c0 + local;
        const uint32_t db = o / m;
        const int64_t g = a.grid_indices[blk0 + db];
        if (g >= 0 && g < a.B) f(j, local, g * a.M + (o - db * m));
    }
}

// Index in the per-cell arrays of cell `local` of chunk `chunk`, -1 for a bad row.
__device__ __forceinline__ int64_t cell_of_chunk(const McDev& a, int64_t chunk, uint32_t local,
                                                 int64_t& g, int64_t& c) {
    const int64_t base = chunk * kChunk;
    const int64_t blk0 = base / a.M;
    const uint32_t m = static_cast<uint32_t>(a.M);
    const uint32_t o = static_cast<uint32_t>(base - blk0 * a.M) + local;
    const uint32_t db = o / m;
    g = a.grid_indices[blk0 + db];
    c = o - db * m;
    return (g >= 0 && g < a.B) ? g * a.M + c : -1;
}

template <int VEC>
__global__ __launch_bounds__(kBlock) void mc_clear_kernel(McDev a) {
    if (blockIdx.x == 0 && threadIdx.x < 4) a.counters[threadIdx.x] = 0;
    const int64_t chunks = (a.n_grids * a.M + kChunk - 1) / kChunk;
    for (int64_t ch = blockIdx.x; ch < chunks; ch += gridDim.x) {
        for_own_groups<VEC>(a, ch, [&](int, uint32_t, int64_t at) {
            if constexpr (VEC == 4) {
                *reinterpret_cast<uint32_t*>(a.cases + at) = 0u;
                *reinterpret_cast<uint4*>(a.slots + at) = make_uint4(0u, 0u, 0u, 0u);
            } else {
                a.cases[at] = 0;
                a.slots[at] = 0u;
            }
        });
    }
}

// Case and flags of a cell whose eight corners are at[0..7].
__device__ __forceinline__ void record_case(const McDev& a, int code, const int64_t* at) {
    a.cases[at[0]] = static_cast<uint8_t>(code);
#pragma unroll
    for (int e = 0; e < 12; ++e) {
        if (edge_crossed(code, e)) flag_edge(a, at[edge_low_corner(e)], e >> 2);
    }
}

// One wavefront per block, blocks taken along the listing (block_walk below).
// tile[] holds, for the (G+1)^3 cells at the corners of the block's cells,
// bit 0 = exists and weighs enough, bit 1 = below the iso value.  Where each tile cell comes from -- the
// block itself or one of its seven neighbours, and which cell there -- is the
// same for every block and is worked out once per workgroup from the tables:
// a cell on a high face of the block names the cells beyond that face.  The
// rows of the next block's neighbours are fetched while the current block is
// processed, so that one block costs one round trip to memory.
constexpr int kTileThreads = 64;
constexpr int kTileMaxGrid = 8192;
constexpr uint16_t kSrcNone = 0xFFFF;   // tile cell that no table entry names
constexpr int kSrcOwn = 8;              // source "the block itself"

__host__ __device__ inline int tile_cells(int g) { return (g + 1) * (g + 1) * (g + 1); }

// s_src[t]: where tile cell t comes from, source << 12 | cell (source 0..7 =
// entry of the block's neighbour row, kSrcOwn = the block itself); s_pos[c]:
// tile index of the block's cell c.
__device__ __forceinline__ void build_tile_map(const McDev& a, uint16_t* s_src, uint16_t* s_pos) {
    const int G = a.g;
    const int W = G + 1;
    const int M = static_cast<int>(a.M);
    const int W3 = tile_cells(G);
    const int lane = threadIdx.x;
    const int off[3] = {1, W, W * W};
    for (int t = lane; t < W3; t += kTileThreads) s_src[t] = kSrcNone;
    __syncthreads();
    for (int c = lane; c < M; c += kTileThreads) {
        int p = 0;
        int high = 0;
#pragma unroll
        for (int d = 0; d < 3; ++d) {
            int x = a.cell_coords[c * 3 + d];
            x = x < 0 ? 0 : (x >= G ? G - 1 : x);
            p += x * off[d];
            high |= (x == G - 1) << d;
        }
        s_pos[c] = static_cast<uint16_t>(p);
        s_src[p] = static_cast<uint16_t>((kSrcOwn << 12) | c);
        for (int nb = 1; nb < 8; ++nb) {
            if (nb & ~high) continue;
            const int64_t gn = a.lut_c2g[c * 8 + nb];
            const int64_t ci = a.lut_c2c[c * 8 + nb];
            if (gn < 0 || gn >= 8 || ci < 0 || ci >= M) continue;
            s_src[p + (nb & 1) + ((nb >> 1) & 1) * W + (nb >> 2) * W * W] =
                    static_cast<uint16_t>((gn << 12) | ci);
        }
    }
}

// The listing positions a one-wavefront workgroup walks.  Workgroups go to the
// eight XCDs round robin and every XCD has an L2 of its own, so each XCD takes
// a contiguous eighth of the listing: with blocks listed in a space-filling
// order, the cells a block fetches from its neighbours have then mostly just
// been fetched by a workgroup on the same XCD.
constexpr int kXcds = 8;

struct BlockWalk {
    int64_t first, end, step;
};

__device__ __forceinline__ BlockWalk block_walk(int64_t n) {
    BlockWalk w;
    if (gridDim.x % kXcds != 0) {
        w.first = blockIdx.x;
        w.end = n;
        w.step = gridDim.x;
        return w;
    }
    const int64_t share = (n + kXcds - 1) / kXcds;
    const int64_t xcd = blockIdx.x % kXcds;
    w.first = xcd * share + blockIdx.x / kXcds;
    w.end = (xcd + 1) * share < n ? (xcd + 1) * share : n;
    w.step = gridDim.x / kXcds;
    return w;
}

// Row of listed block b (lane kSrcOwn) and of its neighbours (lanes 0..7); -1
// where there is none or b is past `end`.
__device__ __forceinline__ int64_t fetch_block_rows(const McDev& a, int64_t b, int64_t end) {
    const int lane = threadIdx.x;
    if (b >= end || lane > kSrcOwn) return -1;
    const int64_t g = a.grid_indices[b];
    if (g < 0 || g >= a.B) return -1;
    if (lane == kSrcOwn) return g;
    const int64_t r = a.lut_g[g * 8 + lane];
    return (r >= 0 && r < a.B) ? r : -1;
}

// Index in the per-cell arrays of tile cell t, -1 if it does not exist.
// s_nb[s]: index of the first cell of source block s (its row times the cells
// per block, multiplied once per block instead of once per tile cell), -1 if
// there is no such block.
__device__ __forceinline__ int64_t tile_source(const uint16_t* s_src, const int64_t* s_nb, int t) {
    const int src = s_src[t];
    const int from = src >> 12;
    if (from > kSrcOwn || s_nb[from] < 0) return -1;
    return s_nb[from] + (src & 0xFFF);
}

template <typename T>
__global__ __launch_bounds__(kTileThreads) void mc_classify_tile_kernel(McDev a) {
    extern __shared__ __align__(16) uint8_t lds[];
    __shared__ int64_t s_nb[kSrcOwn + 1];
    const T* sdfs = static_cast<const T*>(a.sdfs);
    const T* weights = static_cast<const T*>(a.weights);
    const int W = a.g + 1;
    const int M = static_cast<int>(a.M);
    const int W3 = tile_cells(a.g);
    uint32_t* s_list = reinterpret_cast<uint32_t*>(lds);        // [2 * 64] cells the surface crosses
    uint16_t* s_src = reinterpret_cast<uint16_t*>(s_list + 2 * kTileThreads);  // [W3]
    uint16_t* s_pos = s_src + W3;                               // [M]
    uint8_t* tile = reinterpret_cast<uint8_t*>(s_pos + M);      // [W3]
    const int lane = threadIdx.x;
    build_tile_map(a, s_src, s_pos);
    const BlockWalk walk = block_walk(a.n_grids);
    int64_t blk = walk.first;
    int64_t row = fetch_block_rows(a, blk, walk.end);
    for (; blk < walk.end; blk += walk.step) {
        __syncthreads();  // set-up done; previous block's tile, rows and list read
        if (lane <= kSrcOwn) s_nb[lane] = row < 0 ? -1 : row * a.M;
        row = fetch_block_rows(a, blk + walk.step, walk.end);
        __syncthreads();
        if (s_nb[kSrcOwn] < 0) continue;  // the same for the whole wavefront
        for (int t0 = 0; t0 < W3; t0 += 4 * kTileThreads) {
            int64_t at[4];
            T w[4], v[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int t = t0 + k * kTileThreads + lane;
                at[k] = t < W3 ? tile_source(s_src, s_nb, t) : -1;
                w[k] = at[k] >= 0 ? weights[at[k]] : T(0);
                v[k] = at[k] >= 0 ? sdfs[at[k]] : T(0);
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int t = t0 + k * kTileThreads + lane;
                if (t < W3) {
                    tile[t] = at[k] < 0 ? 0
                                        : ((w[k] >= static_cast<T>(a.weight_thr) ? 1 : 0) |
                                           (v[k] - static_cast<T>(a.iso) < T(0) ? 2 : 0));
                }
            }
        }
        __syncthreads();
        // The cells the surface crosses are few (a twentieth in a block at the
        // surface): they are listed first, cell | case << 12, and then handled
        // by consecutive lanes, instead of by the odd lane of every 64 cells.
        // The list holds two rounds of cells and is worked off when a third
        // might not fit.
        int listed = 0;
        auto work_off = [&]() {
            __syncthreads();
            for (int i = lane; i < listed; i += kTileThreads) {
                const int p = s_pos[s_list[i] & 0xFFF];
                const int code = static_cast<int>(s_list[i] >> 12);
                int64_t at[8];
                bool usable = true;
#pragma unroll
                for (int nb = 0; nb < 8; ++nb) {
                    // every corner has a source and a row, or `ok` would be clear
                    const int src = s_src[p + (nb & 1) + ((nb >> 1) & 1) * W + (nb >> 2) * W * W];
                    const int from = src >> 12;
                    usable = usable && from <= kSrcOwn;
                    at[nb] = s_nb[from <= kSrcOwn ? from : kSrcOwn] + (src & 0xFFF);
                }
                if (usable) record_case(a, code, at);
            }
            __syncthreads();
            listed = 0;
        };
        for (int c0 = 0; c0 < M; c0 += kTileThreads) {
            const int c = c0 + lane;
            int code = 0;
            int ok = 0;
            if (c < M) {
                const int p = s_pos[c];
                ok = 1;
#pragma unroll
                for (int nb = 0; nb < 8; ++nb) {
                    const int v = tile[p + (nb & 1) + ((nb >> 1) & 1) * W + (nb >> 2) * W * W];
                    ok &= v;
                    code |= (v >> 1) << nb;
                }
            }
            const bool crossed = ok && code != 0 && code != 255;
            const uint64_t m = __ballot(crossed);
            if (crossed) {
                s_list[listed + __popcll(m & ((1ull << lane) - 1ull))] =
                        static_cast<uint32_t>(c) | (static_cast<uint32_t>(code) << 12);
            }
            listed += __popcll(m);
            if (listed > kTileThreads) work_off();   // the same for the whole wavefront
        }
        work_off();
    }
}

// The same for grids whose blocks do not fit the tile: every cell fetches its
// corners through the tables.
template <typename T>
__global__ __launch_bounds__(kBlock) void mc_classify_cell_kernel(McDev a) {
    const T* sdfs = static_cast<const T*>(a.sdfs);
    const T* weights = static_cast<const T*>(a.weights);
    const int64_t cells = a.n_grids * a.M;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    for (int64_t item = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; item < cells;
         item += stride) {
        const int64_t g = a.grid_indices[item / a.M];
        const int64_t c = item % a.M;
        if (g < 0 || g >= a.B) continue;
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
            code |= (sdfs[at[nb]] - static_cast<T>(a.iso) < T(0)) << nb;
        }
        if (valid && code != 0 && code != 255) record_case(a, code, at);
    }
}

// The case tables in LDS: looked up per cell by every lane, which from global
// memory costs a divergent load each time.
struct McTables {
    uint64_t rows[256];
    uint8_t count[256];
};

__device__ __forceinline__ void load_tables(McTables& t) {
    for (int i = threadIdx.x; i < 256; i += kBlock) {
        t.rows[i] = kMcPackedRows[i];
        t.count[i] = static_cast<uint8_t>(kMcTriangleCount[i]);
    }
    __syncthreads();
}

// Packs the byte flags of classify into bits 0..2 and counts them.
__device__ __forceinline__ uint32_t pack_flags(uint32_t w) {
    return (w & 1u) | ((w >> 7) & 2u) | ((w >> 14) & 4u);
}

template <int VEC>
__global__ __launch_bounds__(kBlock) void mc_count_kernel(McDev a) {
    __shared__ McTables tables;
    load_tables(tables);
    const int64_t chunks = (a.n_grids * a.M + kChunk - 1) / kChunk;
    for (int64_t ch = blockIdx.x; ch < chunks; ch += gridDim.x) {
        int nv = 0;
        int nt = 0;
        for_own_groups<VEC>(a, ch, [&](int, uint32_t, int64_t at) {
            if constexpr (VEC == 4) {
                uint4 w = *reinterpret_cast<const uint4*>(a.slots + at);
                if ((w.x | w.y | w.z | w.w) != 0u) {
                    w = make_uint4(pack_flags(w.x), pack_flags(w.y), pack_flags(w.z),
                                   pack_flags(w.w));
                    *reinterpret_cast<uint4*>(a.slots + at) = w;
                    nv += __popc(w.x) + __popc(w.y) + __popc(w.z) + __popc(w.w);
                }
                const uint32_t codes = *reinterpret_cast<const uint32_t*>(a.cases + at);
#pragma unroll
                for (int k = 0; k < 4; ++k) nt += tables.count[(codes >> (8 * k)) & 0xFFu];
            } else {
                const uint32_t w = a.slots[at];
                if (w != 0u) {
                    a.slots[at] = pack_flags(w);
                    nv += __popc(pack_flags(w));
                }
                nt += tables.count[a.cases[at]];
            }
        });
        // at most 3 * kChunk vertices and 5 * kChunk triangles: 16 bits each
        int total;
        block_exclusive(nv | (nt << 16), total);
        if (threadIdx.x == 0) {
            a.counters[kMcHeader + ch] = total & 0xFFFF;
            a.counters[kMcHeader + chunks + ch] = static_cast<int>(static_cast<uint32_t>(total) >> 16);
        }
    }
}

// Turns `arrays` (1 or 2) consecutive arrays of per-chunk counts into running
// sums (one workgroup; every thread takes a contiguous share of the chunks) and
// stores their totals in ws[slot0] / ws[slot1].
constexpr int kScanThreads = 1024;

__global__ __launch_bounds__(kScanThreads) void mc_scan_kernel(int32_t* ws, int64_t chunks,
                                                              int arrays, int slot0, int slot1) {
    __shared__ int64_t s_sum[kScanThreads];
    const int64_t share = (chunks + kScanThreads - 1) / kScanThreads;
    const int64_t lo = share * threadIdx.x < chunks ? share * threadIdx.x : chunks;
    const int64_t hi = lo + share < chunks ? lo + share : chunks;
    for (int which = 0; which < arrays; ++which) {
        int32_t* counts = ws + kMcHeader + which * chunks;
        int64_t mine = 0;
#pragma unroll 8
        for (int64_t i = lo; i < hi; ++i) mine += counts[i];   // independent loads
        __syncthreads();
        s_sum[threadIdx.x] = mine;
        __syncthreads();
        for (int d = 1; d < kScanThreads; d <<= 1) {
            const int64_t up = threadIdx.x >= d ? s_sum[threadIdx.x - d] : 0;
            __syncthreads();
            s_sum[threadIdx.x] += up;
            __syncthreads();
        }
        int64_t run = s_sum[threadIdx.x] - mine;
#pragma unroll 8
        for (int64_t i = lo; i < hi; ++i) {
            const int32_t n = counts[i];
            counts[i] = static_cast<int32_t>(run < 0x7FFFFFFF ? run : 0x7FFFFFFF);
            run += n;
        }
        if (threadIdx.x == kScanThreads - 1) {
            const int64_t total = s_sum[threadIdx.x];
            ws[which == 0 ? slot0 : slot1] =
                    static_cast<int32_t>(total < 0x7FFFFFFF ? total : 0x7FFFFFFF);
        }
    }
}

// The zero crossings on the flagged +x/+y/+z edges (bits of f) of cell c of row
// g, linear between the two ends of an edge, to positions[out...]
// (ash/src/grid.cu:510-527 and :748-771).
template <typename T>
__device__ __forceinline__ void write_edge_points(const McDev& a, bool standard, int64_t g,
                                                  int64_t c, int64_t own, int f, int64_t out) {
    const T* sdfs = static_cast<const T*>(a.sdfs);
    const T self = sdfs[own] - static_cast<T>(a.iso);
    CellAt at = {0, 0, 0};
    if (standard) {
        at = cell_at(a.g, static_cast<int>(c));
    } else {
        at.x = a.cell_coords[c * 3];
        at.y = a.cell_coords[c * 3 + 1];
        at.z = a.cell_coords[c * 3 + 2];
    }
    const int cell[3] = {at.x, at.y, at.z};
    float base[3];
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        base[d] = static_cast<float>(a.grid_coords[g * 3 + d] * a.g + cell[d]);
    }
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        if (!(f & (1 << d))) continue;
        int64_t gi, ci;
        float ratio = 0.f;
        if (standard ? corner_cell_standard(a, g, at, 1 << d, gi, ci)
                     : corner_cell(a, g, c, 1 << d, gi, ci)) {
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

// Writes the point of every flagged edge: the zero crossing of the field
// along the edge, linear between its two ends (ash/src/grid.cu:510-527 and
// :748-771).  SLOTS: the flags are the low bits of the cells' slot words
// (marching cubes), and every flagged cell's word also receives the id of its
// first point; otherwise they are the low bits of the cells' bytes in `cases`
// (iso-surface points).
template <typename T, int VEC, bool SLOTS>
__global__ __launch_bounds__(kBlock) void edge_points_kernel(McDev a) {
    __shared__ uint16_t s_cell[kChunk];   // cell of the chunk | flags << 12
    __shared__ uint16_t s_id[kChunk];     // its first point, from the chunk's first
    const int64_t chunks = (a.n_grids * a.M + kChunk - 1) / kChunk;
    const bool standard = a.counters[kMcStandard] != 0;
    for (int64_t ch = blockIdx.x; ch < chunks; ch += gridDim.x) {
        uint64_t flags = 0;   // 3 bits per own cell
        int part[kPerThread / VEC] = {};   // per group: listed cells | points << 16
        for_own_groups<VEC>(a, ch, [&](int j, uint32_t, int64_t at) {
            uint32_t f[VEC];
            if constexpr (SLOTS && VEC == 4) {
                const uint4 w = *reinterpret_cast<const uint4*>(a.slots + at);
                f[0] = w.x & 7u;
                f[1] = w.y & 7u;
                f[2] = w.z & 7u;
                f[3] = w.w & 7u;
            } else if constexpr (SLOTS) {
                f[0] = a.slots[at] & 7u;
            } else if constexpr (VEC == 4) {
                const uint32_t w = *reinterpret_cast<const uint32_t*>(a.cases + at);
#pragma unroll
                for (int k = 0; k < 4; ++k) f[k] = (w >> (8 * k)) & 7u;
            } else {
                f[0] = a.cases[at] & 7u;
            }
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                flags |= static_cast<uint64_t>(f[k]) << (3 * (j * VEC + k));
                part[j] += (f[k] != 0u) + (__popc(f[k]) << 16);
            }
        });
        const int total = chunk_exclusive(part);
        const int first = a.counters[kMcHeader + ch];
#pragma unroll
        for (int j = 0; j < kPerThread; ++j) {
            const int f = static_cast<int>(flags >> (3 * j)) & 7;
            if (f) {
                int& at = part[j / VEC];
                s_cell[at & 0xFFFF] =
                        static_cast<uint16_t>((own_group_offset<VEC>(j / VEC) + j % VEC) | (f << 12));
                s_id[at & 0xFFFF] = static_cast<uint16_t>(at >> 16);
                at += 1 + (__popc(f) << 16);
            }
        }
        __syncthreads();
        const int listed = total & 0xFFFF;
        for (int q = threadIdx.x; q < listed; q += kBlock) {
            const int f = s_cell[q] >> 12;
            int64_t g, c;
            const int64_t own = cell_of_chunk(a, ch, s_cell[q] & 0xFFF, g, c);
            const int64_t out = static_cast<int64_t>(first) + s_id[q];
            if constexpr (SLOTS) {
                a.slots[own] = static_cast<uint32_t>(f) | (static_cast<uint32_t>(out) << 3);
            }
            if (out + __popc(f) > a.n_vertices) continue;  // never with the counts of classify
            write_edge_points<T>(a, standard, g, c, own, f, out);
        }
    }
}

// Triangles of every cell with a case, as ids of the vertices on its edges
// (ash/src/grid.cu:796-842).  The table rows already have the orientation the
// reference writes: normals point from below the iso value to above it.
template <int VEC>
__global__ __launch_bounds__(kBlock) void mc_triangles_kernel(McDev a) {
    __shared__ uint32_t s_cell[kChunk];   // cell of the chunk | case << 12
    __shared__ uint16_t s_out[kChunk];    // its first triangle, from the chunk's first
    __shared__ McTables tables;
    load_tables(tables);
    const int64_t chunks = (a.n_grids * a.M + kChunk - 1) / kChunk;
    const bool standard = a.counters[kMcStandard] != 0;
    for (int64_t ch = blockIdx.x; ch < chunks; ch += gridDim.x) {
        uint32_t codes[kPerThread / 4] = {};   // one byte per own cell
        for_own_groups<VEC>(a, ch, [&](int j, uint32_t, int64_t at) {
            if constexpr (VEC == 4) {
                codes[j] = *reinterpret_cast<const uint32_t*>(a.cases + at);
            } else {
                codes[j >> 2] |= static_cast<uint32_t>(a.cases[at]) << (8 * (j & 3));
            }
        });
        int part[kPerThread / VEC] = {};   // per group: listed cells | triangles << 16
#pragma unroll
        for (int j = 0; j < kPerThread; ++j) {
            const uint32_t code = (codes[j >> 2] >> (8 * (j & 3))) & 0xFFu;
            part[j / VEC] += (code != 0u) + (tables.count[code] << 16);
        }
        const int total = chunk_exclusive(part);
        const int first = a.counters[kMcHeader + chunks + ch];
#pragma unroll
        for (int j = 0; j < kPerThread; ++j) {
            const uint32_t code = (codes[j >> 2] >> (8 * (j & 3))) & 0xFFu;
            if (code) {
                int& at = part[j / VEC];
                s_cell[at & 0xFFFF] = (own_group_offset<VEC>(j / VEC) + j % VEC) | (code << 12);
                s_out[at & 0xFFFF] = static_cast<uint16_t>(at >> 16);
                at += 1 + (tables.count[code] << 16);
            }
        }
        __syncthreads();
        const int listed = total & 0xFFFF;
        for (int q = threadIdx.x; q < listed; q += kBlock) {
            const int code = static_cast<int>(s_cell[q] >> 12);
            int64_t g, c;
            if (cell_of_chunk(a, ch, s_cell[q] & 0xFFF, g, c) < 0) continue;
            const int mine = tables.count[code];
            const int64_t first_tri = static_cast<int64_t>(first) + s_out[q];
            if (first_tri + mine > a.n_triangles) continue;  // never with the counts of classify
            // rows of the cells at the eight corners, then the id on every crossed edge
            int need = 0;   // corners that own a crossed edge
#pragma unroll
            for (int e = 0; e < 12; ++e) {
                if (edge_crossed(code, e)) need |= 1 << edge_low_corner(e);
            }
            int64_t at[8];
            const CellAt where = cell_at(a.g, static_cast<int>(c));
#pragma unroll
            for (int nb = 0; nb < 8; ++nb) {
                int64_t gi, ci;
                const bool found = ((need >> nb) & 1) &&
                                   (standard ? corner_cell_standard(a, g, where, nb, gi, ci)
                                             : corner_cell(a, g, c, nb, gi, ci));
                at[nb] = found ? gi * a.M + ci : -1;
            }
            int32_t vid[12];
#pragma unroll
            for (int e = 0; e < 12; ++e) {
                const int axis = e >> 2;
                vid[e] = -1;
                if (edge_crossed(code, e) && at[edge_low_corner(e)] >= 0) {
                    const uint32_t slot = a.slots[at[edge_low_corner(e)]];
                    vid[e] = static_cast<int32_t>(slot >> 3) + __popc(slot & ((1u << axis) - 1u));
                }
            }
            const uint64_t row = tables.rows[code];
            for (int t = 0; t < mine; ++t) {
                int32_t* tri = a.triangles + (first_tri + t) * 3;
#pragma unroll
                for (int v = 0; v < 3; ++v) {
                    const int e = static_cast<int>(row >> (4 * (3 * t + v))) & 15;
                    int32_t id = -1;
#pragma unroll
                    for (int k = 0; k < 12; ++k) {
                        if (k == e) id = vid[k];
                    }
                    tri[v] = id;
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Iso-surface points (ash/src/grid.cu:453-602): every listed cell that weighs
// enough looks at its +x, +y, +z neighbours; where the field changes sign
// against a neighbour that weighs enough as well, the zero crossing on that
// edge is a point.  As in the reference a missing neighbour block ends the
// cell's scan, later axes included, and "changes sign" is `self * other < 0`
// evaluated in the field's type.  The reference runs its kernel twice (count,
// fill) with one atomic per point; here the first call leaves the three
// crossing flags of every cell in `cases` and per-chunk counts in the
// workspace, the second writes the points from the chunks' offsets.
template <typename T>
__device__ __forceinline__ int crossing_flags(T self, const T* diff, const uint8_t* state,
                                              int p, const int* off) {
    int f = 0;
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        const int q = p + off[d];
        const int st = state[q];
        if (!(st & 2)) break;
        if (self * diff[q] < T(0) && (st & 1)) f |= 1 << d;
    }
    return f;
}

// One wavefront per block: field minus iso value of the (G+1)^3 corner cells
// in LDS, state bit 0 = weighs enough, bit 1 = exists.
template <typename T>
__global__ __launch_bounds__(kTileThreads) void iso_classify_tile_kernel(McDev a) {
    extern __shared__ __align__(16) uint8_t lds[];
    __shared__ int64_t s_nb[kSrcOwn + 1];
    const T* sdfs = static_cast<const T*>(a.sdfs);
    const T* weights = static_cast<const T*>(a.weights);
    const int W = a.g + 1;
    const int M = static_cast<int>(a.M);
    const int W3 = tile_cells(a.g);
    T* diff = reinterpret_cast<T*>(lds);                       // [W3]
    uint16_t* s_src = reinterpret_cast<uint16_t*>(diff + W3);  // [W3]
    uint16_t* s_pos = s_src + W3;                              // [M]
    uint8_t* state = reinterpret_cast<uint8_t*>(s_pos + M);    // [W3]
    const int lane = threadIdx.x;
    const int off[3] = {1, W, W * W};
    build_tile_map(a, s_src, s_pos);
    const BlockWalk walk = block_walk(a.n_grids);
    int64_t blk = walk.first;
    int64_t row = fetch_block_rows(a, blk, walk.end);
    for (; blk < walk.end; blk += walk.step) {
        __syncthreads();  // set-up done; previous block's tile and rows read
        if (lane <= kSrcOwn) s_nb[lane] = row < 0 ? -1 : row * a.M;
        row = fetch_block_rows(a, blk + walk.step, walk.end);
        __syncthreads();
        const int64_t g = s_nb[kSrcOwn];  // first cell of the block
        if (g < 0) continue;  // the same for the whole wavefront
        for (int t0 = 0; t0 < W3; t0 += 4 * kTileThreads) {
            int64_t at[4];
            T w[4], v[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int t = t0 + k * kTileThreads + lane;
                at[k] = t < W3 ? tile_source(s_src, s_nb, t) : -1;
                w[k] = at[k] >= 0 ? weights[at[k]] : T(0);
                v[k] = at[k] >= 0 ? sdfs[at[k]] : T(0);
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int t = t0 + k * kTileThreads + lane;
                if (t < W3) {
                    diff[t] = v[k] - static_cast<T>(a.iso);
                    state[t] = at[k] < 0 ? 0 : (2 | (w[k] >= static_cast<T>(a.weight_thr) ? 1 : 0));
                }
            }
        }
        __syncthreads();
        for (int c = lane; c < M; c += kTileThreads) {
            const int p = s_pos[c];
            a.cases[g + c] = static_cast<uint8_t>(
                    (state[p] & 1) ? crossing_flags<T>(diff[p], diff, state, p, off) : 0);
        }
    }
}

// The same through the tables, for blocks that do not fit the tile.
template <typename T>
__global__ __launch_bounds__(kBlock) void iso_classify_cell_kernel(McDev a) {
    const T* sdfs = static_cast<const T*>(a.sdfs);
    const T* weights = static_cast<const T*>(a.weights);
    const int64_t cells = a.n_grids * a.M;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    for (int64_t item = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; item < cells;
         item += stride) {
        const int64_t g = a.grid_indices[item / a.M];
        const int64_t c = item % a.M;
        if (g < 0 || g >= a.B) continue;
        int f = 0;
        if (weights[g * a.M + c] >= static_cast<T>(a.weight_thr)) {
            const T self = sdfs[g * a.M + c] - static_cast<T>(a.iso);
#pragma unroll
            for (int d = 0; d < 3; ++d) {
                int64_t gi, ci;
                if (!corner_cell(a, g, c, 1 << d, gi, ci)) break;
                const T other = sdfs[gi * a.M + ci] - static_cast<T>(a.iso);
                if (self * other < T(0) && weights[gi * a.M + ci] >= static_cast<T>(a.weight_thr)) {
                    f |= 1 << d;
                }
            }
        }
        a.cases[g * a.M + c] = static_cast<uint8_t>(f);
    }
}

template <int VEC>
__global__ __launch_bounds__(kBlock) void iso_count_kernel(McDev a) {
    const int64_t chunks = (a.n_grids * a.M + kChunk - 1) / kChunk;
    for (int64_t ch = blockIdx.x; ch < chunks; ch += gridDim.x) {
        int n = 0;
        for_own_groups<VEC>(a, ch, [&](int, uint32_t, int64_t at) {
            if constexpr (VEC == 4) {
                n += __popc(*reinterpret_cast<const uint32_t*>(a.cases + at) & 0x07070707u);
            } else {
                n += __popc(a.cases[at] & 7u);
            }
        });
        int total;
        block_exclusive(n, total);
        if (threadIdx.x == 0) a.counters[kMcHeader + ch] = total;
    }
}

// Groups of four cells can be moved as one word of cases and one 16-byte
// vector of slots when blocks hold a multiple of four cells and both arrays
// are aligned accordingly.
bool vector_access(const McDev& a) {
    return a.M % 4 == 0 && reinterpret_cast<uintptr_t>(a.cases) % 4 == 0 &&
           reinterpret_cast<uintptr_t>(a.slots) % 16 == 0;
}

// Workgroups of a one-wavefront-per-block launch: a multiple of the number of
// XCDs whenever there are that many blocks (see block_walk).
// No more of them than the device holds at once (256 CUs with 160 KB of LDS
// and 32 wavefronts each): workgroups that had to wait for a free CU would
// start on their share of the blocks when the others are done with theirs.
unsigned tile_grid(int64_t num_grids, size_t lds_bytes) {
    const size_t per_group = (lds_bytes + 128 + 1023) / 1024 * 1024;  // + static, allocation unit
    int64_t per_cu = static_cast<int64_t>(160 * 1024 / per_group);
    if (per_cu > 32) per_cu = 32;
    if (per_cu < 1) per_cu = 1;
    const int64_t resident = per_cu * 256 < kTileMaxGrid ? per_cu * 256 : kTileMaxGrid;
    int64_t g = num_grids < resident ? num_grids : resident;
    if (g >= kXcds) g -= g % kXcds;
    return static_cast<unsigned>(g < 1 ? 1 : g);
}

unsigned chunk_grid(int64_t work_items) {
    if (work_items < 1) return 1;
    return static_cast<unsigned>(work_items < kMaxGrid ? work_items : kMaxGrid);
}

int fill_common(McDev& a, const void* sdfs, const int64_t* grid_indices,
                const int32_t* cell_coords, const int64_t* lut_g, const int64_t* lut_c2c,
                const int64_t* lut_c2g, int64_t num_grids, int64_t num_embeddings,
                int64_t cells_per_grid, int grid_dim, float iso_value, int32_t dtype,
                uint8_t* cases, uint32_t* slots, bool with_slots, int32_t* counters) {
    if (dtype != ASH_F32 && dtype != ASH_F64) ASH_FAIL("unknown dtype");
    if (num_grids < 0 || num_embeddings < 1 || cells_per_grid < 1 || grid_dim < 1) {
        ASH_FAIL("surface extraction: bad sizes");
    }
    if (counters == nullptr) ASH_FAIL("surface extraction: null workspace");
    if (num_grids > 0 &&
        (sdfs == nullptr || grid_indices == nullptr || cell_coords == nullptr ||
         lut_g == nullptr || lut_c2c == nullptr || lut_c2g == nullptr || cases == nullptr ||
         (with_slots && slots == nullptr))) {
        ASH_FAIL("null pointer in surface extraction");
    }
    if (cells_per_grid > (int64_t{1} << 24) || num_grids > (int64_t{1} << 40) / cells_per_grid) {
        ASH_FAIL("marching_cubes: too many cells in one call");
    }
    a.sdfs = sdfs;
    a.grid_indices = grid_indices;
    a.cell_coords = cell_coords;
    a.lut_g = lut_g;
    a.lut_c2c = lut_c2c;
    a.lut_c2g = lut_c2g;
    a.cases = cases;
    a.slots = slots;
    a.counters = counters;
    a.n_grids = num_grids;
    a.B = num_embeddings;
    a.M = cells_per_grid;
    a.g = grid_dim;
    a.iso = iso_value;
    return 0;
}

}  // namespace
}  // namespace ash

using namespace ash;

extern "C" {

int64_t ash_marching_cubes_workspace_ints(int64_t num_grids, int64_t cells_per_grid) {
    if (num_grids < 0 || cells_per_grid < 1) return kMcHeader;
    const int64_t chunks = (num_grids * cells_per_grid + kChunk - 1) / kChunk;
    return kMcHeader + 2 * chunks;
}

int ash_marching_cubes_classify(const void* sdfs, const void* weights,
                                const int64_t* grid_indices,
                                const int64_t* lut_grid_nb2grid_idx,
                                const int32_t* cell_coords_table,
                                const int64_t* lut_cell_nb2cell_idx,
                                const int64_t* lut_cell_nb2grid_nb, int64_t num_grids,
                                int64_t num_embeddings, int64_t cells_per_grid, int grid_dim,
                                float iso_value, float weight_thr, int32_t dtype,
                                uint8_t* cases, uint32_t* edge_slots, int32_t* workspace,
                                void* stream) {
    McDev a = {};
    if (fill_common(a, sdfs, grid_indices, cell_coords_table, lut_grid_nb2grid_idx,
                    lut_cell_nb2cell_idx, lut_cell_nb2grid_nb, num_grids, num_embeddings,
                    cells_per_grid, grid_dim, iso_value, dtype, cases, edge_slots, true, workspace)) {
        return 1;
    }
    if (num_grids > 0 && weights == nullptr) ASH_FAIL("null pointer in marching_cubes");
    a.weights = weights;
    a.weight_thr = weight_thr;
    PointerGuard guard;
    ASH_HIP(guard.enter_for(sdfs));
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t cells = num_grids * cells_per_grid;
    const unsigned by_cell = chunk_grid((cells + kBlock - 1) / kBlock);
    const unsigned by_chunk = chunk_grid((cells + kChunk - 1) / kChunk);
    const bool vec = vector_access(a);
    if (vec) {
        mc_clear_kernel<4><<<by_chunk, kBlock, 0, s>>>(a);
    } else {
        mc_clear_kernel<1><<<by_chunk, kBlock, 0, s>>>(a);
    }
    ASH_LAUNCH_CHECK();
    if (num_grids == 0) return 0;
    layout_check_kernel<<<1, kCheckThreads, 0, s>>>(a);   // after the clear of the header
    ASH_LAUNCH_CHECK();
    const bool tiled = grid_dim <= kMaxTileG &&
                       static_cast<int64_t>(grid_dim) * grid_dim * grid_dim == cells_per_grid;
    if (tiled) {
        const size_t lds = static_cast<size_t>(3 * tile_cells(grid_dim)) + 2 * cells_per_grid +
                           8 * kTileThreads;
        const unsigned by_block = tile_grid(num_grids, lds);
        if (dtype == ASH_F32) {
            mc_classify_tile_kernel<float><<<by_block, kTileThreads, lds, s>>>(a);
        } else {
            mc_classify_tile_kernel<double><<<by_block, kTileThreads, lds, s>>>(a);
        }
    } else if (dtype == ASH_F32) {
        mc_classify_cell_kernel<float><<<by_cell, kBlock, 0, s>>>(a);
    } else {
        mc_classify_cell_kernel<double><<<by_cell, kBlock, 0, s>>>(a);
    }
    ASH_LAUNCH_CHECK();
    if (vec) {
        mc_count_kernel<4><<<by_chunk, kBlock, 0, s>>>(a);
    } else {
        mc_count_kernel<1><<<by_chunk, kBlock, 0, s>>>(a);
    }
    ASH_LAUNCH_CHECK();
    mc_scan_kernel<<<1, kScanThreads, 0, s>>>(workspace, (cells + kChunk - 1) / kChunk, 2,
                                              kMcVertices32, kMcTriangles32);
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
                               uint32_t* edge_slots, int32_t* workspace, int64_t n_vertices,
                               int64_t n_triangles, float* positions, int32_t* triangles,
                               void* stream) {
    McDev a = {};
    if (fill_common(a, sdfs, grid_indices, cell_coords_table, lut_grid_nb2grid_idx,
                    lut_cell_nb2cell_idx, lut_cell_nb2grid_nb, num_grids, num_embeddings,
                    cells_per_grid, grid_dim, iso_value, dtype, const_cast<uint8_t*>(cases),
                    edge_slots, true, workspace)) {
        return 1;
    }
    if (n_vertices < 0 || n_triangles < 0) ASH_FAIL("marching_cubes: negative counts");
    if (n_vertices >= kMaxVertices) ASH_FAIL("marching_cubes: more than 2^29 vertices");
    if (n_triangles > 0x7FFFFFFFll / 3) ASH_FAIL("marching_cubes: too many triangles");
    if (num_grids == 0 || (n_vertices == 0 && n_triangles == 0)) return 0;
    if (grid_coords_table == nullptr || (n_vertices > 0 && positions == nullptr) ||
        (n_triangles > 0 && triangles == nullptr)) {
        ASH_FAIL("null pointer in marching_cubes");
    }
    a.grid_coords = grid_coords_table;
    a.positions = positions;
    a.triangles = triangles;
    a.n_vertices = n_vertices;
    a.n_triangles = n_triangles;
    PointerGuard guard;
    ASH_HIP(guard.enter_for(sdfs));
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t cells = num_grids * cells_per_grid;
    const unsigned by_chunk = chunk_grid((cells + kChunk - 1) / kChunk);
    const bool vec = vector_access(a);
    if (dtype == ASH_F32) {
        if (vec) {
            edge_points_kernel<float, 4, true><<<by_chunk, kBlock, 0, s>>>(a);
        } else {
            edge_points_kernel<float, 1, true><<<by_chunk, kBlock, 0, s>>>(a);
        }
    } else if (vec) {
        edge_points_kernel<double, 4, true><<<by_chunk, kBlock, 0, s>>>(a);
    } else {
        edge_points_kernel<double, 1, true><<<by_chunk, kBlock, 0, s>>>(a);
    }
    ASH_LAUNCH_CHECK();
    if (n_triangles > 0) {
        if (vec) {
            mc_triangles_kernel<4><<<by_chunk, kBlock, 0, s>>>(a);
        } else {
            mc_triangles_kernel<1><<<by_chunk, kBlock, 0, s>>>(a);
        }
        ASH_LAUNCH_CHECK();
    }
    return 0;
}

int64_t ash_isosurface_workspace_ints(int64_t num_grids, int64_t cells_per_grid) {
    if (num_grids < 0 || cells_per_grid < 1) return kMcHeader;
    return kMcHeader + (num_grids * cells_per_grid + kChunk - 1) / kChunk;
}

int ash_isosurface_classify(const void* sdfs, const void* weights, const int64_t* grid_indices,
                            const int64_t* lut_grid_nb2grid_idx,
                            const int32_t* cell_coords_table,
                            const int64_t* lut_cell_nb2cell_idx,
                            const int64_t* lut_cell_nb2grid_nb, int64_t num_grids,
                            int64_t num_embeddings, int64_t cells_per_grid, int grid_dim,
                            float iso_value, float weight_thr, int32_t dtype, uint8_t* flags,
                            int32_t* workspace, void* stream) {
    McDev a = {};
    if (fill_common(a, sdfs, grid_indices, cell_coords_table, lut_grid_nb2grid_idx,
                    lut_cell_nb2cell_idx, lut_cell_nb2grid_nb, num_grids, num_embeddings,
                    cells_per_grid, grid_dim, iso_value, dtype, flags, nullptr, false,
                    workspace)) {
        return 1;
    }
    if (num_grids > 0 && weights == nullptr) ASH_FAIL("null pointer in isosurface_classify");
    a.weights = weights;
    a.weight_thr = weight_thr;
    PointerGuard guard;
    ASH_HIP(guard.enter_for(sdfs));
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t cells = num_grids * cells_per_grid;
    const int64_t chunks = (cells + kChunk - 1) / kChunk;
    if (num_grids > 0) {
        layout_check_kernel<<<1, kCheckThreads, 0, s>>>(a);
        ASH_LAUNCH_CHECK();
        const size_t cell_bytes = dtype == ASH_F32 ? 4 : 8;
        const size_t lds = (cell_bytes + 3) * tile_cells(grid_dim < 64 ? grid_dim : 64) +
                           2 * static_cast<size_t>(cells_per_grid);
        // the tile has to fit the 64 KB a launch may take without further ado
        const bool tiled = grid_dim <= kMaxTileG && lds <= 63 * 1024 &&
                           static_cast<int64_t>(grid_dim) * grid_dim * grid_dim == cells_per_grid;
        if (tiled) {
            const unsigned by_block = tile_grid(num_grids, lds);
            if (dtype == ASH_F32) {
                iso_classify_tile_kernel<float><<<by_block, kTileThreads, lds, s>>>(a);
            } else {
                iso_classify_tile_kernel<double><<<by_block, kTileThreads, lds, s>>>(a);
            }
        } else {
            const unsigned by_cell = chunk_grid((cells + kBlock - 1) / kBlock);
            if (dtype == ASH_F32) {
                iso_classify_cell_kernel<float><<<by_cell, kBlock, 0, s>>>(a);
            } else {
                iso_classify_cell_kernel<double><<<by_cell, kBlock, 0, s>>>(a);
            }
        }
        ASH_LAUNCH_CHECK();
        if (a.M % 4 == 0 && reinterpret_cast<uintptr_t>(flags) % 4 == 0) {
            iso_count_kernel<4><<<chunk_grid(chunks), kBlock, 0, s>>>(a);
        } else {
            iso_count_kernel<1><<<chunk_grid(chunks), kBlock, 0, s>>>(a);
        }
        ASH_LAUNCH_CHECK();
    }
    mc_scan_kernel<<<1, kScanThreads, 0, s>>>(workspace, chunks, 1, 0, 0);
    ASH_LAUNCH_CHECK();
    return 0;
}

int ash_isosurface_points(const void* sdfs, const int64_t* grid_indices,
                          const int32_t* grid_coords_table,
                          const int64_t* lut_grid_nb2grid_idx,
                          const int32_t* cell_coords_table,
                          const int64_t* lut_cell_nb2cell_idx,
                          const int64_t* lut_cell_nb2grid_nb, int64_t num_grids,
                          int64_t num_embeddings, int64_t cells_per_grid, int grid_dim,
                          float iso_value, int32_t dtype, const uint8_t* flags,
                          const int32_t* workspace, int64_t n_points, float* positions,
                          void* stream) {
    McDev a = {};
    if (fill_common(a, sdfs, grid_indices, cell_coords_table, lut_grid_nb2grid_idx,
                    lut_cell_nb2cell_idx, lut_cell_nb2grid_nb, num_grids, num_embeddings,
                    cells_per_grid, grid_dim, iso_value, dtype, const_cast<uint8_t*>(flags),
                    nullptr, false, const_cast<int32_t*>(workspace))) {
        return 1;
    }
    if (n_points < 0 || n_points > 0x7FFFFFFFll) ASH_FAIL("isosurface_points: bad point count");
    if (num_grids == 0 || n_points == 0) return 0;
    if (grid_coords_table == nullptr || positions == nullptr) {
        ASH_FAIL("null pointer in isosurface_points");
    }
    a.grid_coords = grid_coords_table;
    a.positions = positions;
    a.n_vertices = n_points;
    PointerGuard guard;
    ASH_HIP(guard.enter_for(sdfs));
    hipStream_t s = static_cast<hipStream_t>(stream);
    const unsigned by_chunk = chunk_grid((num_grids * cells_per_grid + kChunk - 1) / kChunk);
    const bool vec = a.M % 4 == 0 && reinterpret_cast<uintptr_t>(flags) % 4 == 0;
    if (dtype == ASH_F32) {
        if (vec) {
            edge_points_kernel<float, 4, false><<<by_chunk, kBlock, 0, s>>>(a);
        } else {
            edge_points_kernel<float, 1, false><<<by_chunk, kBlock, 0, s>>>(a);
        }
    } else if (vec) {
        edge_points_kernel<double, 4, false><<<by_chunk, kBlock, 0, s>>>(a);
    } else {
        edge_points_kernel<double, 1, false><<<by_chunk, kBlock, 0, s>>>(a);
    }
    ASH_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
