// Hash map of libash_hip.so: a bucketed open-addressing table for gfx950.
//
// Layout.  A bucket is one 128-byte line holding ten 64-bit key codes followed
// by their ten int32 indices, so a lookup that hits touches one line.  A key
// int32[dim] is packed into a 64-bit code (dim 1: 32 bits, dim 2: 2x32 biased,
// dim 3: 3x21 biased, dim 4: 4x16 biased); a slot is claimed with one 64-bit
// compare-and-swap of the code, which is also what makes duplicate keys inside
// one batch collapse without locks.  Keys whose components do not fit the code
// ("exotic" keys) live in a second, lock-based open-addressing region that is
// only attached once such a key shows up.
//
// Probing.  A wavefront takes 64 keys.  Each group of 8 lanes owns 8 of them
// and probes them one after the other: the 8 lanes read the 8 x 16 bytes of
// the key's bucket in one coalesced request, compare, and agree through
// ballots.  All 8 bucket reads of a group are issued before the first compare,
// so a wavefront keeps 64 lines in flight.  If the bucket neither holds the key
// nor an empty slot the key moves on to the next bucket.
//
// Index allocation follows the reference's heap protocol
// (ash/src/hashmap_gpu.cuh:211-232,316-336): a new key takes heap[counter++],
// an erased key stores its index at heap[--counter]; here the counter is
// advanced once per 256-thread block instead of once per key.
#include "ash_probe.h"

#include "../../include/ash_hip.h"

#include <mutex>

// Scratch of ash_grid_activate_static, the entry point that allocates nothing:
// the list of run heads that ash_grid_activate keeps in a caller-provided
// temporary (one counter line + three int32 per position).  Every device that
// loads the library holds its own copy until the process ends.  In host code
// this name is only a handle for hipGetSymbolAddress; kernels are given the
// address that call returned for the current device.
constexpr int64_t kActivateStaticMax = ASH_ACTIVATE_STATIC_MAX_POSITIONS;
static __device__ __align__(256) int32_t scratch[64 + 3 * kActivateStaticMax];

namespace ash {

static thread_local std::string g_last_error;
void set_error(const std::string& msg) { g_last_error = msg; }

namespace {

constexpr int kBlock = 256;
// Workgroup size of the kernels that advance the heap counter (once per
// workgroup).  Larger groups mean fewer updates of that single address but
// make every wavefront wait for the slowest probe of the group; measured on
// 16 M keys: 256 -> 1.28 ms, 512 -> 1.46 ms, 1024 -> 1.42 ms.
constexpr int kHeapBlock = 256;
constexpr uint32_t kSpinLimit = 1u << 22;

__device__ __forceinline__ uint32_t spread8(uint32_t x) {
    x = (x | (x << 4)) & 0x0F0Fu;
    x = (x | (x << 2)) & 0x3333u;
    x = (x | (x << 1)) & 0x5555u;
    return x;
}

// -------------------------------------------------- cooperative probe pass
enum { kProbeFound = 0, kProbeHasEmpty = 1, kProbeFull = 2 };

struct ProbeResult {
    int status;      // kProbe*
    int slot;        // matching slot (status == kProbeFound)
    int32_t val;     // index stored with the matching slot
    uint32_t emask;  // bit s set <=> slot s was empty in this snapshot
};

// Every lane of the wavefront calls this together.  Lane L owns key L; in
// round r the 8 lanes of a group read the bucket `b` of the group's r-th key
// (16 bytes per lane) and the result lands in that key's owner lane.  Keys
// that are not pending cost no memory traffic.
__device__ __forceinline__ void probe_pass(const MapDev& m, uint64_t code,
                                           uint32_t b, bool pend, int lane,
                                           ProbeResult& out) {
    const int j = lane & (kGroup - 1);
    const int gbase = lane & ~(kGroup - 1);
    const bool v0 = (2 * j) < kSlots;
    const bool v1 = (2 * j + 1) < kSlots;

    uint4 line[kGroup];
#pragma unroll
    for (int r = 0; r < kGroup; ++r) {
        const int src = gbase | r;
        const uint32_t br = __shfl(b, src);
        const int pr = __shfl(static_cast<int>(pend), src);
        line[r] = make_uint4(0u, 0u, 0u, 0u);
        if (pr) {
            line[r] = *(reinterpret_cast<const uint4*>(
                                m.buckets +
                                static_cast<size_t>(br) * kBucketQwords) +
                        j);
        }
    }

#pragma unroll
    for (int r = 0; r < kGroup; ++r) {
        const int src = gbase | r;
        const uint64_t cr = __shfl(code, src);
        const uint64_t qa =
                static_cast<uint64_t>(line[r].x) |
                (static_cast<uint64_t>(line[r].y) << 32);
        const uint64_t qb =
                static_cast<uint64_t>(line[r].z) |
                (static_cast<uint64_t>(line[r].w) << 32);
        const uint32_t gm0 =
                static_cast<uint32_t>(__ballot(v0 && qa == cr) >> gbase) & 0xFFu;
        const uint32_t gm1 =
                static_cast<uint32_t>(__ballot(v1 && qb == cr) >> gbase) & 0xFFu;
        const uint32_t ge0 =
                static_cast<uint32_t>(__ballot(v0 && qa == kEmpty) >> gbase) &
                0xFFu;
        const uint32_t ge1 =
                static_cast<uint32_t>(__ballot(v1 && qb == kEmpty) >> gbase) &
                0xFFu;
        int slot = -1;
        if (gm0) {
            slot = 2 * __builtin_ctz(gm0);
        } else if (gm1) {
            slot = 2 * __builtin_ctz(gm1) + 1;
        }
        const uint32_t emask = spread8(ge0) | (spread8(ge1) << 1);
        const int t = kValDword0 + (slot < 0 ? 0 : slot);
        const int comp = t & 3;
        const uint32_t sel = comp == 0   ? line[r].x
                             : comp == 1 ? line[r].y
                             : comp == 2 ? line[r].z
                                         : line[r].w;
        const int32_t val = __shfl(static_cast<int>(sel), gbase + (t >> 2));
        if (j == r) {
            out.status = slot >= 0 ? kProbeFound
                                   : (emask ? kProbeHasEmpty : kProbeFull);
            out.slot = slot;
            out.val = val;
            out.emask = emask;
        }
    }
}

// ------------------------------------------------ general (exotic) region
enum { kGenWon = 0, kGenDup = 1, kGenFull = 2, kGenNoRegion = 3 };

// Claims a slot for an exotic key.  The slot word goes EMPTY -> LOCKED ->
// NOINDEX (key readable); the caller later stores the index.  A thread that
// meets LOCKED re-reads the word; the holder finishes its few stores inside
// the same loop trip, and the wait is bounded by kSpinLimit.
template <int DIM>
__device__ int gen_claim(const MapDev& m, const int32_t (&k)[DIM],
                         uint32_t& pos) {
    if (m.gstate == nullptr) return kGenNoRegion;
    const uint32_t mask = m.gslots - 1;
    uint32_t p = gen_home<DIM>(k, m.gslots);
    uint32_t step = 0;
    uint32_t spins = 0;
    int result = kGenFull;
    bool done = false;
    while (!done) {
        int32_t w = gen_load(m.gstate + p);
        if (w == kGenEmpty) {
            const int32_t old = atomicCAS(m.gstate + p, kGenEmpty, kGenLocked);
            if (old == kGenEmpty) {
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    __hip_atomic_store(
                            m.gkeys + static_cast<size_t>(p) * 4 + d,
                            d < DIM ? k[d < DIM ? d : 0] : 0, __ATOMIC_RELAXED,
                            __HIP_MEMORY_SCOPE_AGENT);
                }
                __hip_atomic_store(m.gstate + p, kGenNoIndex, __ATOMIC_RELEASE,
                                   __HIP_MEMORY_SCOPE_AGENT);
                pos = p;
                result = kGenWon;
                done = true;
                w = kGenNoIndex;
            } else {
                w = old;
            }
        }
        if (!done) {
            if (w == kGenLocked) {
                if (++spins >= kSpinLimit) done = true;  // give up: kGenFull
            } else {
                if (w != kGenTomb && w != kGenEmpty) {
                    __atomic_thread_fence(__ATOMIC_ACQUIRE);
                    if (gen_key_equal<DIM>(m, p, k)) {
                        result = kGenDup;
                        done = true;
                    }
                }
                if (!done && w != kGenEmpty) {
                    p = (p + 1) & mask;
                    if (++step >= m.gslots) done = true;
                }
            }
        }
    }
    return result;
}

// ------------------------------------------------------------- kernels
// Looks key `k` up; every lane of the wavefront calls this together, lanes
// with active == false only help.  Returns whether the key is stored and, if
// so, its index in `res`.
template <int DIM>
__device__ __forceinline__ bool find_key(const MapDev& m, const int32_t (&k)[DIM],
                                         bool active, int32_t& res) {
    const int lane = threadIdx.x & 63;
    uint64_t code;
    const bool fits = pack_key<DIM>(k, code);
    bool pend = active && fits;
    uint32_t b = bucket_of(code, m.nb);
    uint32_t steps = 0;
    res = 0;
    bool found = false;
    while (__ballot(pend)) {
        ProbeResult p;
        probe_pass(m, code, b, pend, lane, p);
        if (pend) {
            if (p.status == kProbeFound) {
                found = true;
                res = p.val;
                pend = false;
            } else if (p.status == kProbeHasEmpty) {
                pend = false;
            } else {
                b = next_bucket(b, m.nb);
                if (++steps >= kPartBuckets) pend = false;
            }
        }
    }
    if (active && !fits) {
        uint32_t pos;
        found = gen_find<DIM>(m, k, res, pos);
    }
    return found;
}

// The same look-up when the eight lanes of a group all hold the same key (and
// the same `active`): the group reads the key's bucket once, 16 bytes per lane,
// instead of taking turns with eight different keys.
template <int DIM>
__device__ __forceinline__ bool find_key_shared(const MapDev& m, const int32_t (&k)[DIM],
                                                bool active, int32_t& res) {
    const int lane = threadIdx.x & 63;
    const int j = lane & (kGroup - 1);
    const int gbase = lane & ~(kGroup - 1);
    const bool v0 = (2 * j) < kSlots;
    const bool v1 = (2 * j + 1) < kSlots;
    uint64_t code;
    const bool fits = pack_key<DIM>(k, code);
    bool pend = active && fits;
    uint32_t b = bucket_of(code, m.nb);
    uint32_t steps = 0;
    res = 0;
    bool found = false;
    while (__ballot(pend)) {
        uint4 line = make_uint4(0u, 0u, 0u, 0u);
        if (pend) {
            line = *(reinterpret_cast<const uint4*>(m.buckets +
                                                    static_cast<size_t>(b) * kBucketQwords) + j);
        }
        const uint64_t qa = static_cast<uint64_t>(line.x) | (static_cast<uint64_t>(line.y) << 32);
        const uint64_t qb = static_cast<uint64_t>(line.z) | (static_cast<uint64_t>(line.w) << 32);
        const uint32_t gm0 = static_cast<uint32_t>(__ballot(pend && v0 && qa == code) >> gbase) & 0xFFu;
        const uint32_t gm1 = static_cast<uint32_t>(__ballot(pend && v1 && qb == code) >> gbase) & 0xFFu;
        const uint32_t ge0 = static_cast<uint32_t>(__ballot(pend && v0 && qa == kEmpty) >> gbase) & 0xFFu;
        const uint32_t ge1 = static_cast<uint32_t>(__ballot(pend && v1 && qb == kEmpty) >> gbase) & 0xFFu;
        int slot = -1;
        if (gm0) {
            slot = 2 * __builtin_ctz(gm0);
        } else if (gm1) {
            slot = 2 * __builtin_ctz(gm1) + 1;
        }
        const int t = kValDword0 + (slot < 0 ? 0 : slot);
        const int comp = t & 3;
        const uint32_t sel = comp == 0 ? line.x : comp == 1 ? line.y : comp == 2 ? line.z : line.w;
        const int32_t val = __shfl(static_cast<int>(sel), gbase + (t >> 2));
        if (pend) {
            if (slot >= 0) {
                found = true;
                res = val;
                pend = false;
            } else if (ge0 | ge1) {
                pend = false;
            } else {
                b = next_bucket(b, m.nb);
                if (++steps >= kPartBuckets) pend = false;
            }
        }
    }
    if (active && !fits) {
        uint32_t pos;
        found = gen_find<DIM>(m, k, res, pos);
    }
    return found;
}

template <int DIM>
__global__ __launch_bounds__(kBlock) void find_kernel(
        MapDev m, const int32_t* __restrict__ keys, int64_t n,
        int64_t* __restrict__ idx_out, uint8_t* __restrict__ mask_out) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const bool active = i < n;
    int32_t k[DIM];
    load_key<DIM>(keys, i, active, k);
    int32_t res = 0;
    const bool found = find_key<DIM>(m, k, active, res);
    if (active) {
        idx_out[i] = found ? static_cast<int64_t>(res) : 0;
        mask_out[i] = found ? 1 : 0;
    }
}

// Fused front end of the sparse-dense grid query (ash/grid.py:183-199): splits a
// position x (cell units) into block / cell / fractional part (split_axis) and
// looks the block up (find_block_by_runs), in one pass.
__global__ __launch_bounds__(kBlock) void grid_query_kernel(
        MapDev m, const float* __restrict__ x, int64_t n, float g, int gi,
        int64_t* __restrict__ grid_idx, int64_t* __restrict__ cell_idx,
        float* __restrict__ off, uint8_t* __restrict__ mask_out) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const bool active = i < n;
    int32_t k[3];
    float o[3];
    int64_t cell = 0;
    int64_t stride = 1;
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        int32_t c;
        split_axis(active ? x[i * 3 + d] : 0.f, g, k[d], c, o[d]);
        cell += static_cast<int64_t>(c) * stride;
        stride *= gi;
    }
    int32_t res = 0;
    const bool found = find_block_by_runs(m, k, active, res);
    if (active) {
        grid_idx[i] = found ? static_cast<int64_t>(res) : 0;
        mask_out[i] = found ? 1 : 0;
        cell_idx[i] = cell;
        off[i * 3 + 0] = o[0];
        off[i * 3 + 1] = o[1];
        off[i * 3 + 2] = o[2];
    }
}

enum InsertMode {
    kInsertKeys = 0,    // allocate indices only
    kInsertFused = 1,   // + copy narrow value rows in the same kernel
    kInsertAssign = 2,  // + report the allocated index per input row
    kInsertLoad = 3,    // indices are given (state-dict load), heap untouched
    kInsertReport = 4   // keys only; tells the caller the key's index when it is final
};

// The insert proper for a key held in registers (`code` is its packed form if
// `fits`); `i` is the row of the key's value rows / `assigned` / `given` entry.
template <int DIM, int MODE>
__device__ __forceinline__ void insert_key(
        const MapDev& m, const int32_t (&k)[DIM], uint64_t code, bool fits,
        int64_t i, bool active, const ValueArgs& va,
        int32_t* __restrict__ assigned, const int64_t* __restrict__ given,
        int32_t* report = nullptr) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    int32_t seen = -1;     // kInsertReport: the index read beside a key that was there
    bool gdup = false;     // kInsertReport: the key stands in the general region
    bool pend = active && fits;
    uint32_t b = bucket_of(code, m.nb);
    uint32_t steps = 0;

    bool won = false;      // claimed a packed slot (wb, ws)
    bool gwon = false;     // claimed a general slot gp
    bool refused = false;  // no room anywhere
    uint32_t wb = 0, gp = 0;
    int ws = 0;

    // Phase A: claim a slot per new key.
    while (__ballot(pend)) {
        ProbeResult p;
        probe_pass(m, code, b, pend, lane, p);
        if (pend) {
            if (p.status == kProbeFound) {
                pend = false;
                if constexpr (MODE == kInsertLoad) {
                    atomicAdd(m.ctr + kCtrLoadDup, 1);
                }
                if constexpr (MODE == kInsertReport) seen = p.val;
            } else {
                uint32_t em = p.emask;
                while (em) {
                    const int s = __builtin_ctz(em);
                    const unsigned long long old =
                            atomicCAS(slot_ptr(m, b, s), kEmpty, code);
                    if (old == kEmpty) {
                        won = true;
                        wb = b;
                        ws = s;
                        pend = false;
                        break;
                    }
                    if (old == code) {
                        pend = false;
                        if constexpr (MODE == kInsertLoad) {
                            atomicAdd(m.ctr + kCtrLoadDup, 1);
                        }
                        break;
                    }
                    em &= em - 1;
                }
                if (pend) {
                    b = next_bucket(b, m.nb);
                    if (++steps >= kPartBuckets) {
                        pend = false;
                        refused = true;
                    }
                }
            }
        }
    }
    if (active && !fits) {
        const int g = gen_claim<DIM>(m, k, gp);
        if (g == kGenWon) {
            gwon = true;
        } else if (g == kGenFull) {
            refused = true;
        } else if (g == kGenNoRegion) {
            atomicAdd(m.ctr + kCtrExotic, 1);
        } else if constexpr (MODE == kInsertLoad) {
            atomicAdd(m.ctr + kCtrLoadDup, 1);
        } else if constexpr (MODE == kInsertReport) {
            gdup = true;
        }
    }
    if (refused) atomicAdd(m.ctr + kCtrDropped, 1);

    // Phase B: one heap-counter update per block, indices for the winners.
    const bool w = won || gwon;
    int32_t idx = -1;
    if constexpr (MODE == kInsertLoad) {
        if (w) {
            // the index comes with the key (`given` null: the key's own number,
            // when the keys are the entries of the key log)
            const int64_t g = given != nullptr ? given[i] : i;
            if (g >= 0 && g < m.capacity) {
                idx = static_cast<int32_t>(g);
            } else {
                // an index that addresses no row: the pair is refused (the
                // slot goes back) and counted with the duplicates
                if (won) {
                    atomicExch(slot_ptr(m, wb, ws), kTomb);
                } else {
                    __hip_atomic_store(m.gstate + gp, kGenTomb, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                    atomicAdd(m.ctr + kCtrGenTombs, 1);
                }
                atomicAdd(m.ctr + kCtrTombs, 1);
                atomicAdd(m.ctr + kCtrLoadDup, 1);
            }
        }
    } else {
        __shared__ int s_cnt[kHeapBlock / 64];
        __shared__ int s_base;
        const uint64_t wm = __ballot(w);
        const int nw = __popcll(wm);
        const int rank = __popcll(wm & ((1ull << lane) - 1ull));
        if (lane == 0) s_cnt[wave] = nw;
        __syncthreads();
        if (threadIdx.x == 0) {
            int tot = 0;
#pragma unroll
            for (int q = 0; q < kHeapBlock / 64; ++q) tot += s_cnt[q];
            int base = 0;
            if (tot > 0) {
                base = atomicAdd(m.ctr + kCtrSize, tot);
                if (base + tot > m.capacity) {
                    const int lo = base > m.capacity ? base : m.capacity;
                    const int excess = base + tot - lo;
                    atomicSub(m.ctr + kCtrSize, excess);
                    atomicAdd(m.ctr + kCtrDropped, excess);
                }
            }
            s_base = base;
        }
        __syncthreads();
        int top = s_base + rank;
        for (int q = 0; q < wave; ++q) top += s_cnt[q];
        if (w) {
            if (top < m.capacity) {
                idx = m.heap[top];
                // (a heap that a state dict brought may hold anything: an entry
                // that addresses no row is treated like an exhausted heap)
                if (static_cast<uint32_t>(idx) >= static_cast<uint32_t>(m.capacity)) idx = -1;
            }
            if (idx < 0) {
                // Heap exhausted: give the slot up again.
                if (won) {
                    atomicExch(slot_ptr(m, wb, ws), kTomb);
                } else {
                    __hip_atomic_store(m.gstate + gp, kGenTomb,
                                       __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                    atomicAdd(m.ctr + kCtrGenTombs, 1);
                }
                atomicAdd(m.ctr + kCtrTombs, 1);
            }
        }
    }
    if (idx >= 0) {
        // (0 <= idx < capacity: heap entries are, loaded indices were checked)
        if (won) {
            *value_ptr(m, wb, ws) = idx;
            m.klog[idx] = code;
        } else {
            __hip_atomic_store(m.gstate + gp, idx, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
            m.klog[idx] = kTomb;   // "stored in the general region"
            atomicAdd(m.ctr + kCtrGenLive, 1);
        }
        if constexpr (MODE == kInsertFused) {
#pragma unroll
            for (int v = 0; v < kMaxFusedValues; ++v) {
                if (v < va.n) {
                    const int rd = va.row_dwords[v];
                    const uint32_t* s = va.src[v] + i * rd;
                    uint32_t* d = va.dst[v] + static_cast<int64_t>(idx) * rd;
                    for (int q = 0; q < rd; ++q) d[q] = s[q];
                }
            }
        }
    }
    if constexpr (MODE == kInsertAssign) {
        if (active) assigned[i] = idx;
    }
    if constexpr (MODE == kInsertReport) {
        // The index of the key, if this thread can be sure of it: the one it
        // was given just now, or the one read beside a key that was there --
        // but a key that another thread is storing in this very launch shows
        // before its index is written, and the word beside it still holds
        // whatever an earlier tenant of the slot left.  The key log settles
        // it: klog[index] names this key only if that index is the key's own.
        // (-1 tells the caller that the thread storing the key will know.)
        int32_t r = idx;
        if (r < 0 && static_cast<uint32_t>(seen) < static_cast<uint32_t>(m.capacity) &&
            m.klog[seen] == code) {
            r = seen;
        }
        if (r < 0 && gdup) {
            // (the general region shows an index only once it is final)
            uint32_t at;
            int32_t gi;
            if (gen_find<DIM>(m, k, gi, at)) r = gi;
        }
        *report = r;
    }
}

// One key per thread, every thread of the workgroup calls this together.
// CODES: `keys` holds packed 64-bit codes instead of int32[DIM] rows.
template <int DIM, int MODE, bool CODES>
__device__ __forceinline__ void insert_one(
        const MapDev& m, const int32_t* __restrict__ keys, int64_t i,
        bool active, const ValueArgs& va, int32_t* __restrict__ assigned,
        const int64_t* __restrict__ given) {
    int32_t k[DIM] = {};
    uint64_t code;
    bool fits;
    if constexpr (CODES) {
        code = active ? reinterpret_cast<const uint64_t*>(keys)[i] : 0ull;
        fits = true;
    } else {
        load_key<DIM>(keys, i, active, k);
        fits = pack_key<DIM>(k, code);
    }
    insert_key<DIM, MODE>(m, k, code, fits, i, active, va, assigned, given);
}

template <int DIM, int MODE>
__global__ __launch_bounds__(kHeapBlock) void insert_kernel(
        MapDev m, const int32_t* __restrict__ keys, int64_t n, ValueArgs va,
        int32_t* __restrict__ assigned, const int64_t* __restrict__ given) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kHeapBlock + threadIdx.x;
    insert_one<DIM, MODE, false>(m, keys, i, i < n, va, assigned, given);
}

// The same insert over a selection made on the device: thread t of the
// selection handles row sel[t], t < *nsel.  The grid is fixed; workgroups
// stride over the selection, which is empty in the common case.
template <int DIM, int MODE, bool CODES>
__global__ __launch_bounds__(kHeapBlock) void insert_selected_kernel(
        MapDev m, const int32_t* __restrict__ keys,
        const int32_t* __restrict__ sel, const int32_t* __restrict__ nsel,
        ValueArgs va) {
    const int64_t total = *nsel;
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * kHeapBlock;
         base < total; base += static_cast<int64_t>(gridDim.x) * kHeapBlock) {
        const int64_t t = base + threadIdx.x;
        const bool active = t < total;
        const int64_t i = active ? sel[t] : 0;
        insert_one<DIM, MODE, CODES>(m, keys, i, active, va, nullptr, nullptr);
        __syncthreads();
    }
}

// Block activation around a batch of positions (ash/grid.py:121-159): the
// block of every position and its neighbours within the dilation are inserted
// as int3 keys.  The reference expands every position into (2r+1)^3 candidate
// rows, de-duplicates them through a scratch hash set and inserts the
// survivors.  Here positions arrive in image order, so their blocks come in
// runs: activate_heads_kernel keeps one block per run ("head", one atomic per
// wavefront to reserve list space), and activate_kernel then handles one
// (head, neighbour offset) pair per thread, the table absorbing the remaining
// duplicates.  MARK = false inserts; MARK = true (a second launch, when every
// index is final) looks the candidates up again, flags their rows in `touched`
// and records their coordinates, from which the caller lists the touched
// blocks.
__device__ __forceinline__ bool block_of_position(
        const float* __restrict__ cells, int64_t i, float g, int bound_lo,
        int bound_hi, int32_t (&base)[3]) {
    bool inside = true;
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        base[d] = static_cast<int32_t>(floorf(__fdiv_rn(cells[i * 3 + d], g)));
        inside = inside && base[d] >= bound_lo && base[d] <= bound_hi;
    }
    return inside;
}

// heads[0] = number of heads (zero on entry), heads[64 + 3 h ..] = block h.
// One update of the shared counter per 1024 positions.
constexpr int kHeadsBlock = 1024;

__global__ __launch_bounds__(kHeadsBlock) void activate_heads_kernel(
        const float* __restrict__ cells, int64_t n, float g, int bound_lo,
        int bound_hi, int32_t* __restrict__ heads) {
    __shared__ int s_cnt[kHeadsBlock / 64];
    __shared__ int s_first;
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kHeadsBlock + threadIdx.x;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    int32_t base[3] = {0, 0, 0};
    bool lead = false;
    if (i < n) {
        lead = block_of_position(cells, i, g, bound_lo, bound_hi, base);
        if (lead && i > 0) {
            int32_t prev[3];
            const bool pin = block_of_position(cells, i - 1, g, bound_lo, bound_hi, prev);
            lead = !pin || prev[0] != base[0] || prev[1] != base[1] || prev[2] != base[2];
        }
    }
    const uint64_t lm = __ballot(lead);
    if (lane == 0) s_cnt[wave] = __popcll(lm);
    __syncthreads();
    if (threadIdx.x == 0) {
        int tot = 0;
#pragma unroll
        for (int q = 0; q < kHeadsBlock / 64; ++q) {
            const int c = s_cnt[q];
            s_cnt[q] = tot;
            tot += c;
        }
        s_first = tot ? atomicAdd(heads, tot) : 0;
    }
    __syncthreads();
    if (lead) {
        int32_t* out = heads + 64 +
                       3 * static_cast<int64_t>(s_first + s_cnt[wave] +
                                                __popcll(lm & ((1ull << lane) - 1ull)));
        out[0] = base[0];
        out[1] = base[1];
        out[2] = base[2];
    }
}

template <bool MARK>
__global__ __launch_bounds__(kHeapBlock) void activate_kernel(
        MapDev m, const int32_t* __restrict__ heads, int off_lo, int width,
        int bound_lo, int bound_hi, uint8_t* __restrict__ touched,
        int32_t* __restrict__ coords) {
    const int per_head = width * width * width;
    const int64_t total = static_cast<int64_t>(heads[0]) * per_head;
    const ValueArgs none = {};
    for (int64_t first = static_cast<int64_t>(blockIdx.x) * kHeapBlock; first < total;
         first += static_cast<int64_t>(gridDim.x) * kHeapBlock) {
        const int64_t t = first + threadIdx.x;
        bool ok = t < total;
        int32_t k[3] = {0, 0, 0};
        if (ok) {
            const int64_t h = t / per_head;
            const int o = static_cast<int>(t - h * per_head);
            const int32_t* base = heads + 64 + 3 * h;
            k[0] = base[0] + off_lo + o % width;
            k[1] = base[1] + off_lo + (o / width) % width;
            k[2] = base[2] + off_lo + o / (width * width);
#pragma unroll
            for (int d = 0; d < 3; ++d) {
                ok = ok && k[d] >= bound_lo && k[d] <= bound_hi;
            }
        }
        if constexpr (!MARK) {
            uint64_t code;
            const bool fits = pack_key<3>(k, code);
            insert_key<3, kInsertKeys>(m, k, code, fits, 0, ok, none, nullptr, nullptr);
            __syncthreads();
        } else {
            int32_t idx = 0;
            const bool found = find_key<3>(m, k, ok, idx);
            if (found && ok) {
                touched[idx] = 1;
                coords[static_cast<int64_t>(idx) * 3 + 0] = k[0];
                coords[static_cast<int64_t>(idx) * 3 + 1] = k[1];
                coords[static_cast<int64_t>(idx) * 3 + 2] = k[2];
            }
        }
    }
}

// The same activation straight from world positions, without a list of run
// heads in memory: a workgroup finds the heads among its own kRunPositions
// positions (a position leads a run when the position before it lies in
// another block, whichever workgroup that one belongs to), keeps them in LDS
// and handles their (head, neighbour offset) pairs itself: no list to write
// and read back, no counter to clear.
// Positions are in world units: cell units = (x - origin) * inv_cell, evaluated
// as torch evaluates `(x - origin) / cell_size` on the device (grid_forward's
// front end does the same); origin null and inv_cell 1 leave them as they are.
struct RunsArgs {
    const float* x;        // float32[n, 3]
    const float* origin;   // float32[3] on the device, or nullptr
    float inv_cell;
    float g;               // cells per block edge
    int64_t n;
    int off_lo, width;     // neighbour offsets off_lo .. off_lo + width - 1 per axis
    int bound_lo, bound_hi;
};

__device__ __forceinline__ bool block_of_world(const RunsArgs& a, int64_t i,
                                               int32_t (&base)[3]) {
    bool inside = true;
#pragma unroll
    for (int d = 0; d < 3; ++d) {
        const float o = a.origin != nullptr ? a.origin[d] : 0.f;
        const float c = __fmul_rn(__fsub_rn(a.x[i * 3 + d], o), a.inv_cell);
        base[d] = static_cast<int32_t>(floorf(__fdiv_rn(c, a.g)));
        inside = inside && base[d] >= a.bound_lo && base[d] <= a.bound_hi;
    }
    return inside;
}

constexpr int kRunPositions = 256;
static_assert(kRunPositions % 64 == 0 && kRunPositions <= kHeapBlock, "whole wavefronts of positions");
constexpr int kCandChunk = 1024;         // candidates made distinct at a time
constexpr int kDistinctSlots = 2048;     // two LDS slots per candidate of a chunk

// One launch per batch: insert and flag.  The (head, neighbour offset)
// candidates of a workgroup -- some 270 for 128 depth pixels at dilation 1 --
// name every block twice on average (the neighbourhoods of neighbouring
// blocks overlap in 18 of 27), so they are first made distinct in an LDS set,
// which leaves one round of table work per workgroup as a rule.  The insert
// reports the index of every key it can be sure of (insert_key, kInsertReport)
// and the row is flagged at once; a key that another thread is storing at
// that moment is flagged by that thread, which is handed the index.  No second
// launch has to wait for the indices to settle.
__global__ __launch_bounds__(kHeapBlock) void activate_runs_kernel(
        MapDev m, RunsArgs a, uint8_t* __restrict__ touched, int32_t* __restrict__ coords) {
    __shared__ unsigned long long s_set[kDistinctSlots];
    __shared__ int32_t s_cand[kCandChunk * 3];
    __shared__ int32_t s_heads[kRunPositions * 3];
    __shared__ int s_wave[kRunPositions / 64];
    __shared__ int s_ncand;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kRunPositions + threadIdx.x;
    int32_t base[3] = {0, 0, 0};
    bool lead = false;
    if (threadIdx.x < kRunPositions && i < a.n) {
        lead = block_of_world(a, i, base);
        if (lead && i > 0) {
            int32_t prev[3];
            const bool pin = block_of_world(a, i - 1, prev);
            lead = !pin || prev[0] != base[0] || prev[1] != base[1] || prev[2] != base[2];
        }
    }
    const uint64_t lm = __ballot(lead);
    if (lane == 0 && wave < kRunPositions / 64) s_wave[wave] = __popcll(lm);
    __syncthreads();
    int before = 0, nh = 0;
#pragma unroll
    for (int q = 0; q < kRunPositions / 64; ++q) {
        const int c = s_wave[q];
        if (q < wave) before += c;
        nh += c;
    }
    if (lead) {
        const int h = before + __popcll(lm & ((1ull << lane) - 1ull));
        s_heads[h * 3 + 0] = base[0];
        s_heads[h * 3 + 1] = base[1];
        s_heads[h * 3 + 2] = base[2];
    }
    const int per_head = a.width * a.width * a.width;
    const int total = nh * per_head;   // the same for every thread of the workgroup
    const ValueArgs none = {};
    for (int first = 0; first < total; first += kCandChunk) {
        for (int q = threadIdx.x; q < kDistinctSlots; q += kHeapBlock) s_set[q] = kEmpty;
        if (threadIdx.x == 0) s_ncand = 0;
        __syncthreads();   // (also: s_heads is complete, the rounds below are over)
        const int end = total - first < kCandChunk ? total : first + kCandChunk;
        for (int t = first + threadIdx.x; t < end; t += kHeapBlock) {
            const int h = t / per_head;
            const int o = t - h * per_head;
            int32_t c[3];
            c[0] = s_heads[h * 3 + 0] + a.off_lo + o % a.width;
            c[1] = s_heads[h * 3 + 1] + a.off_lo + (o / a.width) % a.width;
            c[2] = s_heads[h * 3 + 2] + a.off_lo + o / (a.width * a.width);
            bool keep = true;
#pragma unroll
            for (int d = 0; d < 3; ++d) keep = keep && c[d] >= a.bound_lo && c[d] <= a.bound_hi;
            uint64_t code;
            if (keep && pack_key<3>(c, code)) {   // (keys that do not pack are all kept)
                uint32_t at = static_cast<uint32_t>(mix64(code)) & (kDistinctSlots - 1);
                for (;;) {   // at most half of the slots are ever taken
                    const unsigned long long old = atomicCAS(&s_set[at], kEmpty, code);
                    if (old == kEmpty) break;
                    if (old == code) {
                        keep = false;
                        break;
                    }
                    at = (at + 1) & (kDistinctSlots - 1);
                }
            }
            if (keep) {
                const int at = atomicAdd(&s_ncand, 1);
                s_cand[at * 3 + 0] = c[0];
                s_cand[at * 3 + 1] = c[1];
                s_cand[at * 3 + 2] = c[2];
            }
        }
        __syncthreads();
        const int distinct = s_ncand;
        for (int r0 = 0; r0 < distinct; r0 += kHeapBlock) {
            const int t = r0 + threadIdx.x;
            const bool ok = t < distinct;
            int32_t k[3] = {0, 0, 0};
            if (ok) {
                k[0] = s_cand[t * 3 + 0];
                k[1] = s_cand[t * 3 + 1];
                k[2] = s_cand[t * 3 + 2];
            }
            uint64_t code;
            const bool fits = pack_key<3>(k, code);
            int32_t row = -1;
            insert_key<3, kInsertReport>(m, k, code, fits, 0, ok, none, nullptr, nullptr, &row);
            if (ok && row >= 0) {
                touched[row] = 1;
                coords[static_cast<int64_t>(row) * 3 + 0] = k[0];
                coords[static_cast<int64_t>(row) * 3 + 1] = k[1];
                coords[static_cast<int64_t>(row) * 3 + 2] = k[2];
            }
            __syncthreads();   // insert_key's own words are rewritten by the next round
        }
    }
}

// --------------------------------------------------------------------- rays
// ash/src/sampler.cu:7-67 and :122-214.  Positions are
// origin + t * direction as a fused multiply-add (what nvcc makes of the
// reference's expression); everything is in cell units and a block is
// `grid2cell` cells wide.
__device__ __forceinline__ void ray_block(const float (&o)[3], const float (&d)[3],
                                          float t, float cell2grid,
                                          int32_t (&block)[3], float (&x)[3]) {
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        x[a] = fmaf(t, d[a], o[a]);
        block[a] = static_cast<int32_t>(floorf(__fmul_rn(x[a], cell2grid)));
    }
}

// One wavefront per ray: the march of ray_find_near_far visits the parameters
// t_0 = t_min, t_{k+1} = t_k + step regardless of what it finds, so lane l of
// round r takes step 64 r + l (its t by the same chain of additions), the 64
// lookups go out together, and the near / far recurrence is then replayed over
// the hits in step order.  The march ends at the first step that is at or
// beyond t_max or outside the box, exactly where the sequential loop stops.
__global__ __launch_bounds__(kBlock) void ray_near_far_kernel(
        MapDev m, const float* __restrict__ origins,
        const float* __restrict__ directions, const float* __restrict__ bbox_min,
        const float* __restrict__ bbox_max, int64_t n, float t_min, float t_max,
        float grid2cell, float* __restrict__ nears, float* __restrict__ fars) {
    const int lane = threadIdx.x & 63;
    const int64_t i = static_cast<int64_t>(blockIdx.x) * (kBlock / 64) + (threadIdx.x >> 6);
    if (i >= n) return;  // whole wavefronts leave together
    const float cell2grid = static_cast<float>(1.0 / grid2cell);
    const float t_grid_step = static_cast<float>(grid2cell * 0.5);
    float o[3], d[3], lo[3], hi[3];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        o[a] = origins[i * 3 + a];
        d[a] = directions[i * 3 + a];
        lo[a] = bbox_min[a];
        hi[a] = bbox_max[a];
    }
    float t = t_min;
    for (int j = 0; j < 63; ++j) {
        if (j < lane) t += t_grid_step;
    }
    float near = -1.f, far = t_max;
    for (;;) {
        int32_t block[3];
        float x[3];
        ray_block(o, d, t, cell2grid, block, x);
        bool go = t < t_max;
#pragma unroll
        for (int a = 0; a < 3; ++a) go = go && x[a] >= lo[a] && x[a] <= hi[a];
        const uint64_t stop = __ballot(!go);
        const int first_stop = stop ? __builtin_ctzll(stop) : 64;
        const bool active = lane < first_stop;
        // steps are half a block apart, so neighbouring lanes often stand in
        // the same block: only the first lane of such a run goes to the table,
        // the others take its answer
        bool head = true;
        {
            int same = lane > 0;
#pragma unroll
            for (int a = 0; a < 3; ++a) same &= __shfl_up(block[a], 1) == block[a];
            head = !same;
        }
        int32_t idx;
        const bool asked = find_key_alone<3>(m, block, active && head, idx);
        const uint64_t heads = __ballot(head);
        const int my_head = 63 - __builtin_clzll(heads & (~0ull >> (63 - lane)));
        const bool found = __shfl(static_cast<int>(asked), my_head) != 0;
        uint64_t hits = __ballot(found && active);
        while (hits) {
            const int l = __builtin_ctzll(hits);
            const float t_hit = __shfl(t, l);
            near = near < 0.f ? t_hit : fmaxf(near - t_grid_step, t_min);
            far = fminf(t_hit + t_grid_step, t_max);
            hits &= hits - 1;
        }
        if (first_stop < 64) break;
        for (int j = 0; j < 64; ++j) t += t_grid_step;
    }
    if (lane == 0) {
        nears[i] = near;
        fars[i] = far;
    }
}

// counts != nullptr: allocation pass; otherwise the assignment pass, which
// writes the samples of ray i at prefix[i - 1] .. prefix[i].  An allocation
// pass with `stage` also keeps the first `stride` samples of ray i as pairs
// (t_near, t_far) at stage[2 * (i * stride + k)], so that the assignment pass
// can be a copy instead of a second march.
// LPR lanes per ray: 1 (every lane looks its block up by itself,
// find_key_alone), or 8 lanes that march the same ray in step and share every
// look-up (find_key_shared) -- eight times the wavefronts for the same rays,
// which is what hides the latency of a march that is one dependent look-up
// after the other when the rays are few.
template <int LPR>
__global__ __launch_bounds__(kBlock) void ray_sample_kernel(
        MapDev m, const float* __restrict__ origins,
        const float* __restrict__ directions, const float* __restrict__ ray_nears,
        const float* __restrict__ ray_fars, int64_t n, float max_samples,
        float grid2cell, int64_t* __restrict__ counts,
        const int64_t* __restrict__ prefix, int64_t* __restrict__ ray_indices,
        float* __restrict__ t_nears, float* __restrict__ t_fars,
        float2* __restrict__ stage, int64_t stride) {
    const int64_t gid = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const int64_t i = gid / LPR;
    const bool writer = gid % LPR == 0;   // the lane of a ray that stores its results
    const bool active = i < n;
    const float cell2grid = static_cast<float>(1.0 / grid2cell);
    float o[3], d[3];
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        o[a] = active ? origins[i * 3 + a] : 0.f;
        d[a] = active ? directions[i * 3 + a] : 0.f;
    }
    const float ray_near = active ? ray_nears[i] : 0.f;
    const float ray_far = active ? ray_fars[i] : 0.f;
    const float t_step = fmaxf(0.7f, __fdiv_rn(ray_far - ray_near, max_samples));
    const float t_grid_step = __fmul_rn(t_step, grid2cell);
    const int64_t start = (counts == nullptr && active && i > 0) ? prefix[i - 1] : 0;
    float t = ray_near, t_near = ray_near;
    int64_t local = 0;
    bool live = active && t < ray_far;
    // One step of the march, given whether the block under t is stored.
    auto step = [&](bool found) {
        const float before = t;
        if (!found) {
            t += t_grid_step;
        } else {
            t += t_step;
            if (!writer) {
            } else if (counts == nullptr) {
                ray_indices[start + local] = i;
                t_nears[start + local] = t_near;
                t_fars[start + local] = t;
            } else if (stage != nullptr && local < stride) {
                stage[i * stride + local] = make_float2(t_near, t);
            }
            t_near = t;
            ++local;
        }
        // a step that no longer advances t (range far beyond fp32
        // resolution) would never end; the reference has no such guard
        live = t < ray_far && t > before;
    };
    // The reference looks the block under t up at every step.  Samples are a
    // fraction of a block apart, so consecutive steps mostly ask for the same
    // block: a lane answers those from its last look-up and the wavefront goes
    // to the table only when some lane has entered another block -- a dozen
    // round trips to memory per ray instead of one per step, same answers.
    int32_t known[3] = {0, 0, 0};
    bool have = false;
    bool known_found = false;
    while (__ballot(live)) {
        int32_t block[3] = {0, 0, 0};
        float x[3];
        bool ask = false;
        while (live) {
            ray_block(o, d, t, cell2grid, block, x);
            if (!have || block[0] != known[0] || block[1] != known[1] || block[2] != known[2]) {
                ask = true;
                break;
            }
            step(known_found);
        }
        int32_t idx;
        const bool found = LPR == 8 ? find_key_shared<3>(m, block, live && ask, idx)
                                    : find_key_alone<3>(m, block, live && ask, idx);
        if (live && ask) {
#pragma unroll
            for (int a = 0; a < 3; ++a) known[a] = block[a];
            known_found = found;
            have = true;
            step(found);
        }
    }
    if (active && writer && counts != nullptr) counts[i] = local;
}

// Assignment pass from the staged samples: one thread per staged slot.
__global__ __launch_bounds__(kBlock) void ray_compact_kernel(
        const int64_t* __restrict__ counts, const int64_t* __restrict__ prefix,
        const float2* __restrict__ stage, int64_t stride, int64_t n,
        int64_t* __restrict__ ray_indices, float* __restrict__ t_nears,
        float* __restrict__ t_fars) {
    const int64_t slot = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (slot >= n * stride) return;
    const int64_t i = slot / stride;
    const int64_t k = slot - i * stride;
    if (k >= counts[i]) return;
    const int64_t out = (i > 0 ? prefix[i - 1] : 0) + k;
    const float2 s = stage[slot];
    ray_indices[out] = i;
    t_nears[out] = s.x;
    t_fars[out] = s.y;
}

// Workgroup size of erase: the heap counter and the tombstone counter are each
// updated once per workgroup, and updates of one address serialise (about 7 ns
// each), so larger groups pay off here: measured on 16 M stored keys,
// 256 threads with a tombstone update per wavefront 3.0 ms, 1024 threads with
// one update of each counter per workgroup 0.85 ms.
constexpr int kEraseBlock = 1024;

// One key per thread, every thread of the workgroup calls this together.
// CODES: `keys` holds packed 64-bit codes instead of int32[DIM] rows.
template <int DIM, bool CODES>
__device__ __forceinline__ void erase_one(const MapDev& m, const int32_t* __restrict__ keys,
                                          int64_t i, bool active) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    int32_t k[DIM] = {};
    uint64_t code;
    bool fits;
    if constexpr (CODES) {
        code = active ? reinterpret_cast<const uint64_t*>(keys)[i] : 0ull;
        fits = true;
    } else {
        load_key<DIM>(keys, i, active, k);
        fits = pack_key<DIM>(k, code);
    }
    bool pend = active && fits;
    uint32_t b = bucket_of(code, m.nb);
    uint32_t steps = 0;
    bool won = false;
    bool tomb = false;
    int32_t idx = 0;
    while (__ballot(pend)) {
        ProbeResult p;
        probe_pass(m, code, b, pend, lane, p);
        if (pend) {
            if (p.status == kProbeFound) {
                // A bucket that still has an empty slot has never been full,
                // so no key was ever pushed past it: the slot can go straight
                // back to empty.  Otherwise leave a tombstone.
                const bool reuse = p.emask != 0;
                const unsigned long long old = atomicCAS(
                        slot_ptr(m, b, p.slot), code, reuse ? kEmpty : kTomb);
                if (old == code) {
                    won = true;
                    tomb = !reuse;
                    idx = p.val;
                }
                pend = false;
            } else if (p.status == kProbeHasEmpty) {
                pend = false;
            } else {
                b = next_bucket(b, m.nb);
                if (++steps >= kPartBuckets) pend = false;
            }
        }
    }
    if (active && !fits) {
        int32_t gi;
        uint32_t pos;
        if (gen_find<DIM>(m, k, gi, pos)) {
            if (atomicCAS(m.gstate + pos, gi, kGenTomb) == gi) {
                won = true;
                tomb = true;
                idx = gi;
                atomicSub(m.ctr + kCtrGenLive, 1);
                atomicAdd(m.ctr + kCtrGenTombs, 1);
            }
        }
    }
    __shared__ int s_cnt[kEraseBlock / 64];
    __shared__ int s_tomb[kEraseBlock / 64];
    __shared__ int s_base;
    const uint64_t wm = __ballot(won);
    const int nw = __popcll(wm);
    const int rank = __popcll(wm & ((1ull << lane) - 1ull));
    const int nt = __popcll(__ballot(tomb));
    if (lane == 0) {
        s_cnt[wave] = nw;
        s_tomb[wave] = nt;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int tot = 0, tombs = 0;
#pragma unroll
        for (int q = 0; q < kEraseBlock / 64; ++q) {
            tot += s_cnt[q];
            tombs += s_tomb[q];
        }
        if (tombs > 0) atomicAdd(m.ctr + kCtrTombs, tombs);
        s_base = tot > 0 ? atomicSub(m.ctr + kCtrSize, tot) : 0;
    }
    __syncthreads();
    if (won) {
        int below = rank;
        for (int q = 0; q < wave; ++q) below += s_cnt[q];
        const int pos = s_base - 1 - below;
        if (pos >= 0 && pos < m.capacity) m.heap[pos] = idx;
        if (static_cast<uint32_t>(idx) < static_cast<uint32_t>(m.capacity)) m.klog[idx] = kEmpty;
    }
}

template <int DIM>
__global__ __launch_bounds__(kEraseBlock) void erase_kernel(
        MapDev m, const int32_t* __restrict__ keys, int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kEraseBlock + threadIdx.x;
    erase_one<DIM, false>(m, keys, i, i < n);
}

// The same erase over a selection made on the device (see
// insert_selected_kernel): thread t handles key sel[t], t < *nsel.
template <int DIM, bool CODES>
__global__ __launch_bounds__(kEraseBlock) void erase_selected_kernel(
        MapDev m, const int32_t* __restrict__ keys, const int32_t* __restrict__ sel,
        const int32_t* __restrict__ nsel) {
    const int64_t total = *nsel;
    for (int64_t base = static_cast<int64_t>(blockIdx.x) * kEraseBlock; base < total;
         base += static_cast<int64_t>(gridDim.x) * kEraseBlock) {
        const int64_t t = base + threadIdx.x;
        const bool active = t < total;
        erase_one<DIM, CODES>(m, keys, active ? sel[t] : 0, active);
        __syncthreads();   // the counters in LDS are free again
    }
}

// items(): the live entries are read from the key log (8 bytes per index,
// against 21 bytes per index of bucket array).  A workgroup takes 8192
// consecutive indices, each of its wavefronts 512 of them in eight rounds of
// 64, so that reads are contiguous and -- positions being ranks in index order
// -- so are the writes of every round; the entries of a workgroup come out
// sorted by index, workgroups in the order in which they reserve their output
// range.  `limit` indices are scanned: the capacity, or -- when nothing has
// written to the heap since it was last 0, 1, 2, ... (`identity`) and the
// indices in use therefore are 0 .. size-1 -- only the size.
// Output ranges come from one global cursor; atomics on that single address
// serialise (about 7 ns each across the XCDs), hence the large workgroups.
constexpr int kItemsBlock = 1024;
constexpr int kItemsRounds = 8;
constexpr int kItemsSpan = kItemsBlock * kItemsRounds;   // indices per workgroup

// items() while the heap is in its initial order and no key lives in the
// second region: the indices in use are 0 .. n-1, every one of them, so entry
// i of the output is index i and its key comes from log entry i -- no ranks,
// no cursor, and the value rows of the listed entries are the first n rows of
// every value tensor.
template <int DIM>
__global__ __launch_bounds__(kBlock) void items_dense_kernel(
        MapDev m, int32_t* __restrict__ keys_out, int64_t* __restrict__ idx_out, int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i >= n) return;
    int32_t k[DIM];
    unpack_key<DIM>(m.klog[i], k);
#pragma unroll
    for (int d = 0; d < DIM; ++d) keys_out[i * DIM + d] = k[d];
    idx_out[i] = i;
}

template <int DIM>
__global__ __launch_bounds__(kItemsBlock) void items_kernel(
        MapDev m, int32_t* __restrict__ keys_out, int64_t* __restrict__ idx_out,
        int64_t n_expected, int identity) {
    constexpr int kWaves = kItemsBlock / 64;
    __shared__ int s_cnt[kWaves * kItemsRounds];
    __shared__ int s_base;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t limit = identity ? static_cast<int64_t>(m.ctr[kCtrSize])
                                   : static_cast<int64_t>(m.capacity);
    const int64_t first = static_cast<int64_t>(blockIdx.x) * kItemsSpan;
    if (first >= limit) return;
    const int64_t mine = first + wave * (64 * kItemsRounds) + lane;
    uint64_t code[kItemsRounds];
    int rank[kItemsRounds];
#pragma unroll
    for (int r = 0; r < kItemsRounds; ++r) {
        const int64_t i = mine + r * 64;
        code[r] = i < limit ? m.klog[i] : kEmpty;
        const uint64_t live = __ballot(code[r] < kTomb);
        rank[r] = __popcll(live & ((1ull << lane) - 1ull));
        if (lane == 0) s_cnt[wave * kItemsRounds + r] = __popcll(live);
    }
    __syncthreads();
    // exclusive scan of the 128 counts by the first two wavefronts
    const bool scanner = threadIdx.x < kWaves * kItemsRounds;
    int c = 0, incl = 0;
    if (scanner) {
        c = s_cnt[threadIdx.x];
        incl = c;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(incl, d);
            if (lane >= d) incl += up;
        }
    }
    __syncthreads();
    if (scanner) {
        s_cnt[threadIdx.x] = incl - c;
        if (threadIdx.x == 63) s_base = incl;   // total of the first 64 counts
    }
    __syncthreads();
    if (scanner && threadIdx.x >= 64) s_cnt[threadIdx.x] += s_base;
    __syncthreads();
    if (threadIdx.x == kWaves * kItemsRounds - 1) {
        const int tot = s_cnt[threadIdx.x] + c;
        s_base = tot > 0 ? atomicAdd(m.ctr + kCtrCursor, tot) : 0;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kItemsRounds; ++r) {
        if (code[r] < kTomb) {
            const int64_t pos = static_cast<int64_t>(s_base) + s_cnt[wave * kItemsRounds + r] + rank[r];
            if (pos < n_expected) {
                int32_t k[DIM];
                unpack_key<DIM>(code[r], k);
#pragma unroll
                for (int d = 0; d < DIM; ++d) keys_out[pos * DIM + d] = k[d];
                idx_out[pos] = mine + r * 64;
            }
        }
    }
}

template <int DIM>
__global__ __launch_bounds__(kBlock) void items_general_kernel(
        MapDev m, int32_t* __restrict__ keys_out, int64_t* __restrict__ idx_out,
        int64_t n_expected) {
    const uint32_t p = blockIdx.x * kBlock + threadIdx.x;
    const int lane = threadIdx.x & 63;
    int32_t w = kGenEmpty;
    if (p < m.gslots) w = m.gstate[p];
    const bool live = w >= 0;
    const uint64_t lm = __ballot(live);
    if (lm == 0) return;
    const int rank = __popcll(lm & ((1ull << lane) - 1ull));
    int base = 0;
    if (lane == 0) base = atomicAdd(m.ctr + kCtrCursor, __popcll(lm));
    base = __shfl(base, 0);
    if (live) {
        const int64_t pos = static_cast<int64_t>(base) + rank;
        if (pos < n_expected) {
#pragma unroll
            for (int d = 0; d < DIM; ++d) {
                keys_out[pos * DIM + d] = m.gkeys[static_cast<size_t>(p) * 4 + d];
            }
            idx_out[pos] = w;
        }
    }
}

__global__ __launch_bounds__(kBlock) void fill16_kernel(uint4* __restrict__ p,
                                                        int64_t n16,
                                                        uint32_t word) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    const uint4 v = make_uint4(word, word, word, word);
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
         i < n16; i += stride) {
        p[i] = v;
    }
}

// klog[0 .. limit) := free, limit = the capacity or (prefix_only) the size
// counter -- or, if larger, the index below which an earlier clear left its
// entries standing -- rounded up to whole 16-byte units.  The log's allocation is a
// multiple of 16 bytes plus slack (256-byte aligned workspace regions), so the
// last unit of an odd capacity is written whole.
__global__ __launch_bounds__(kBlock) void empty_log_kernel(
        uint4* __restrict__ log16, int64_t capacity, const int32_t* __restrict__ ctr,
        int prefix_only) {
    int64_t entries = capacity;
    if (prefix_only) {
        const int64_t size = ctr[kCtrSize], high = ctr[kCtrLogHigh];
        const int64_t used = size > high ? size : high;
        entries = used < capacity ? used : capacity;
    }
    const int64_t n16 = (entries + 1) / 2;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    const uint4 v = make_uint4(~0u, ~0u, ~0u, ~0u);
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n16;
         i += stride) {
        log16[i] = v;
    }
}

// klog[size .. kCtrLogHigh) := free (8-byte stores: an odd size shares its
// 16 bytes with an entry in use).
__global__ __launch_bounds__(kBlock) void empty_log_tail_kernel(
        uint64_t* __restrict__ klog, int64_t capacity, const int32_t* __restrict__ ctr) {
    const int64_t from = ctr[kCtrSize] < 0 ? 0 : ctr[kCtrSize];
    const int64_t high = ctr[kCtrLogHigh];
    const int64_t to = high < capacity ? high : capacity;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    for (int64_t i = from + static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < to;
         i += stride) {
        klog[i] = kEmpty;
    }
}

// `keep_log`: the key log is left as it is; the counter kCtrLogHigh then
// remembers how far it may hold entries (the size so far, or what an earlier
// call remembered).
__global__ __launch_bounds__(kBlock) void reset_heap_kernel(
        int32_t* __restrict__ heap, int64_t capacity, int32_t* __restrict__ ctr,
        int32_t size_value, bool write_heap, bool keep_log) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (write_heap && i < capacity) heap[i] = static_cast<int32_t>(i);
    if (i < kNumCounters) {
        // (one wavefront: every lane has read before any lane writes)
        const int32_t size = ctr[kCtrSize], high = ctr[kCtrLogHigh];
        int32_t v = 0;
        if (i == kCtrSize) v = size_value;
        if (i == kCtrLogHigh && keep_log) v = size > high ? size : high;
        ctr[i] = v;
    }
}

// Keys counted as waiting for the second region although it is attached (a
// graph captured before the attach still runs without it) cannot be issued
// again by anybody: they are counted with the refused keys.
__global__ void fold_waiting_keys_kernel(int32_t* ctr) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        ctr[kCtrDropped] += ctr[kCtrExotic];
        ctr[kCtrExotic] = 0;
    }
}

__global__ void set_counter_kernel(int32_t* ctr, int which, int32_t value) {
    if (threadIdx.x == 0 && blockIdx.x == 0) ctr[which] = value;
}

template <typename Unit>
__global__ __launch_bounds__(kBlock) void scatter_rows_kernel(
        const Unit* __restrict__ src, Unit* __restrict__ dst,
        const int32_t* __restrict__ assigned, int64_t n, int64_t units_per_row) {
    const int64_t total = n * units_per_row;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    for (int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
         t < total; t += stride) {
        const int64_t row = t / units_per_row;
        const int64_t u = t - row * units_per_row;
        const int32_t a = assigned[row];
        if (a >= 0) dst[static_cast<int64_t>(a) * units_per_row + u] = src[t];
    }
}

// Row gather for up to kMaxFusedValues tensors at once: word t of output plane
// v is word t % rd of row indices[t / rd] of source plane v.  One launch reads
// the indices once per word of a row (the repeats hit the first-level cache);
// with indices in ascending runs, as items() returns them, source reads are
// contiguous.  RD = row width in words, 0 = read it from the arguments.
struct GatherArgs {
    int n;
    const uint32_t* src[kMaxFusedValues];
    uint32_t* dst[kMaxFusedValues];
    int32_t row_dwords[kMaxFusedValues];
    int64_t src_rows[kMaxFusedValues];
};

template <int RD>
__device__ __forceinline__ void gather_plane(const uint32_t* __restrict__ src,
                                             uint32_t* __restrict__ dst, int rd_runtime,
                                             const int64_t* __restrict__ indices, int64_t n,
                                             int64_t src_rows) {
    const uint32_t rd = RD > 0 ? static_cast<uint32_t>(RD) : static_cast<uint32_t>(rd_runtime);
    const int64_t words = n * rd;
    const bool narrow = words <= 0xFFFFFFFFll;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    for (int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; t < words;
         t += stride) {
        const int64_t row = narrow ? static_cast<int64_t>(static_cast<uint32_t>(t) / rd) : t / rd;
        const uint32_t q = static_cast<uint32_t>(t - row * rd);
        const int64_t from = indices[row];
        // an index outside the source reads as zero instead of faulting
        __builtin_nontemporal_store((from >= 0 && from < src_rows) ? src[from * rd + q] : 0u, dst + t);
    }
}

// The first n rows of every plane, copied: what the gather is while the listing
// has entry i under index i.  16 bytes per thread where both sides allow it;
// source and copy are each touched once (non-temporal hint).
__global__ __launch_bounds__(kBlock) void copy_first_rows_kernel(GatherArgs a, int64_t n) {
    typedef unsigned int v4u __attribute__((ext_vector_type(4)));
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    for (int v = 0; v < a.n; ++v) {
        const uint32_t* __restrict__ src = a.src[v];
        uint32_t* __restrict__ dst = a.dst[v];
        const int64_t have = a.src_rows[v] < n ? a.src_rows[v] : n;   // rows beyond the source read as zero
        const int64_t words = n * a.row_dwords[v];
        const int64_t live = have * a.row_dwords[v];
        const bool wide = reinterpret_cast<uintptr_t>(src) % 16 == 0 &&
                          reinterpret_cast<uintptr_t>(dst) % 16 == 0;
        const int64_t quads = wide ? live / 4 : 0;
        for (int64_t t = tid; t < quads; t += stride) {
            __builtin_nontemporal_store(
                    __builtin_nontemporal_load(reinterpret_cast<const v4u*>(src) + t),
                    reinterpret_cast<v4u*>(dst) + t);
        }
        for (int64_t t = 4 * quads + tid; t < words; t += stride) dst[t] = t < live ? src[t] : 0u;
    }
}

__global__ __launch_bounds__(kBlock) void gather_rows_kernel(
        GatherArgs a, const int64_t* __restrict__ indices, int64_t n) {
    for (int v = 0; v < a.n; ++v) {
        switch (a.row_dwords[v]) {
            case 1:
                gather_plane<1>(a.src[v], a.dst[v], 1, indices, n, a.src_rows[v]);
                break;
            case 2:
                gather_plane<2>(a.src[v], a.dst[v], 2, indices, n, a.src_rows[v]);
                break;
            case 3:
                gather_plane<3>(a.src[v], a.dst[v], 3, indices, n, a.src_rows[v]);
                break;
            case 4:
                gather_plane<4>(a.src[v], a.dst[v], 4, indices, n, a.src_rows[v]);
                break;
            default:
                gather_plane<0>(a.src[v], a.dst[v], a.row_dwords[v], indices, n, a.src_rows[v]);
                break;
        }
    }
}

// The rows whose flag an activation has set, in ascending order, with their
// block coordinates; the flags are cleared on the way and the count goes to
// the table's counters, where the read-back that follows an activation finds
// it (and where ash_grid_integrate_depth_touched reads it on the device).
//
// Up to kCollectGroups workgroups, each with a chunk of the flags: a workgroup
// holds its own chunk in registers (one run of `words` 4-flag words per thread,
// so that thread order is flag order), counts the flags of all chunks before
// its own (they sit in L2: every workgroup reads them) and so knows where its
// rows go without waiting for anybody.  Nobody may clear flags while others
// still count them: each workgroup draws a ticket when it has read all it
// needs, and the one that draws the last ticket clears the whole array and
// puts the ticket counter back to zero.
constexpr int kCollectThreads = 1024;
constexpr int kCollectGroups = 128;
constexpr int kCollectMaxWords = 2;    // per thread: 2^20 flags / 128 groups / 1024 threads / 4
constexpr int64_t kCollectMaxBlocks = int64_t{1} << 20;   // ASH_COLLECT_MAX_BLOCKS of the header

__device__ __forceinline__ int flags_in(uint32_t w) {
    return (w & 0xFFu ? 1 : 0) + (w & 0xFF00u ? 1 : 0) + (w & 0xFF0000u ? 1 : 0) +
           (w & 0xFF000000u ? 1 : 0);
}

// word `i` of the flags, bytes beyond `capacity` read as zero
__device__ __forceinline__ uint32_t flag_word(const uint8_t* touched, int64_t i, int64_t capacity) {
    const int64_t at = i * 4;
    if (at + 4 <= capacity) return *reinterpret_cast<const uint32_t*>(touched + at);
    uint32_t w = 0;
    for (int b = 0; at + b < capacity; ++b) w |= static_cast<uint32_t>(touched[at + b]) << (8 * b);
    return w;
}

// Sum of `v` over the workgroup; `mine` = sum over the threads before this one.
__device__ __forceinline__ int block_sums(int v, int* s_wave, int& mine) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    int incl = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d);
        if (lane >= d) incl += up;
    }
    __syncthreads();   // s_wave free again
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    mine = incl - v;
    int total = 0;
    for (int q = 0; q < kCollectThreads / 64; ++q) {
        if (q < wave) mine += s_wave[q];
        total += s_wave[q];
    }
    return total;
}

__global__ __launch_bounds__(kCollectThreads) void collect_touched_kernel(
        uint8_t* __restrict__ touched, const int32_t* __restrict__ block_coords,
        int64_t capacity, int words, int64_t* __restrict__ out_idx,
        int32_t* __restrict__ out_coords, int32_t* __restrict__ ctr) {
    __shared__ int s_wave[kCollectThreads / 64];
    __shared__ int s_last;
    const int64_t chunk_words = static_cast<int64_t>(words) * kCollectThreads;
    const int64_t first_word = blockIdx.x * chunk_words + static_cast<int64_t>(threadIdx.x) * words;
    uint32_t w[kCollectMaxWords];
    int own = 0;
#pragma unroll
    for (int i = 0; i < kCollectMaxWords; ++i) {
        w[i] = i < words ? flag_word(touched, first_word + i, capacity) : 0u;
        own += flags_in(w[i]);
    }
    int before = 0;
    const int64_t words_before = blockIdx.x * chunk_words;   // whole words, inside the array
    if (reinterpret_cast<uintptr_t>(touched) % 16 == 0) {
        const uint4* quads = reinterpret_cast<const uint4*>(touched);
#pragma unroll 8
        for (int64_t i = threadIdx.x; i < words_before / 4; i += kCollectThreads) {
            const uint4 v = quads[i];
            before += flags_in(v.x) + flags_in(v.y) + flags_in(v.z) + flags_in(v.w);
        }
    } else {
#pragma unroll 8
        for (int64_t i = threadIdx.x; i < words_before; i += kCollectThreads) {
            before += flags_in(reinterpret_cast<const uint32_t*>(touched)[i]);
        }
    }
    int unused;
    const int base = block_sums(before, s_wave, unused);
    int pos;
    const int total = block_sums(own, s_wave, pos);
    pos += base;
    if (threadIdx.x == 0) {
        if (blockIdx.x == gridDim.x - 1) ctr[kCtrTouched] = base + total;
        __threadfence();
        s_last = atomicAdd(ctr + kCtrTicket, 1) == static_cast<int>(gridDim.x) - 1;
    }
#pragma unroll
    for (int i = 0; i < kCollectMaxWords; ++i) {
        if (w[i] == 0u) continue;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            if ((w[i] >> (8 * b)) & 0xFFu) {
                const int64_t at = (first_word + i) * 4 + b;
                out_idx[pos] = at;
                out_coords[pos * 3 + 0] = block_coords[at * 3 + 0];
                out_coords[pos * 3 + 1] = block_coords[at * 3 + 1];
                out_coords[pos * 3 + 2] = block_coords[at * 3 + 2];
                ++pos;
            }
        }
    }
    __syncthreads();
    if (!s_last) return;
    // every workgroup has read what it needs
    const int64_t whole = capacity / 4;
    for (int64_t i = threadIdx.x; i < whole; i += kCollectThreads) {
        reinterpret_cast<uint32_t*>(touched)[i] = 0u;
    }
    if (threadIdx.x < capacity - whole * 4) touched[whole * 4 + threadIdx.x] = 0;
    if (threadIdx.x == 0) ctr[kCtrTicket] = 0;
}

// Puts the entries of the packed region back into an emptied bucket array:
// entry i of the key log is the code stored under index i.  `identity`: only
// the entries below the size are in use (see items_kernel).
__global__ __launch_bounds__(kHeapBlock) void replace_from_log_kernel(MapDev m, int identity) {
    const int64_t limit = identity ? static_cast<int64_t>(m.ctr[kCtrSize])
                                   : static_cast<int64_t>(m.capacity);
    const ValueArgs none = {};
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kHeapBlock;
    for (int64_t first = static_cast<int64_t>(blockIdx.x) * kHeapBlock; first < limit;
         first += stride) {
        const int64_t i = first + threadIdx.x;
        const uint64_t code = i < limit ? m.klog[i] : kEmpty;
        const int32_t k[1] = {0};
        insert_key<1, kInsertLoad>(m, k, code, true, i, code < kTomb, none, nullptr, nullptr);
    }
}

// Entries of a heap that address no row, counted with the pairs a load refuses.
__global__ __launch_bounds__(kBlock) void check_heap_kernel(const int32_t* __restrict__ heap,
                                                           int64_t capacity,
                                                           int32_t* __restrict__ ctr) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    int bad = 0;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < capacity;
         i += stride) {
        bad += static_cast<uint32_t>(heap[i]) >= static_cast<uint32_t>(capacity) ? 1 : 0;
    }
    if (bad) atomicAdd(ctr + kCtrLoadDup, bad);
}

// ---------------------------------------------------------------- host
inline unsigned grid_for(int64_t n, int per_block = kBlock) {
    return static_cast<unsigned>((n + per_block - 1) / per_block);
}

// One unit per thread as far as a launch goes (the kernels loop beyond that):
// workgroups that are handed out one after the other walk through memory in
// order, which the memory side rewards (a 1.6 GB fill: 6.8 TB/s, against 5.7
// with 16 384 workgroups that stride through it and 4.5 with 4096).
inline unsigned capped_grid(int64_t n) {
    int64_t g = (n + kBlock - 1) / kBlock;
    const int64_t cap = 0x7FFFFFFF;
    if (g > cap) g = cap;
    if (g < 1) g = 1;
    return static_cast<unsigned>(g);
}

// For the kernels that move rows by index (random on one side): 8192
// workgroups that loop (one unit per thread: 0.23 against 0.185 ms for the 16 M
// rows of two value tensors).
inline unsigned looping_grid(int64_t n) {
    int64_t g = (n + kBlock - 1) / kBlock;
    const int64_t cap = 256 * 32;
    if (g > cap) g = cap;
    if (g < 1) g = 1;
    return static_cast<unsigned>(g);
}

// Few rays cannot fill the device with one lane each; below this many they
// march with eight lanes per ray (32 768 rays: 110 against 120 us; from 65 536
// rays on one lane per ray is the faster one, 1.6x at half a million).
constexpr int64_t kRaysPerLaneMin = int64_t{1} << 16;

int launch_ray_sample(ash_map_t* map, const float* origins, const float* directions,
                      const float* nears, const float* fars, int64_t n, float max_samples,
                      float grid2cell, int64_t* counts, const int64_t* prefix,
                      int64_t* ray_indices, float* t_nears, float* t_fars, float2* stage,
                      int64_t stride, hipStream_t s) {
    if (n < kRaysPerLaneMin) {
        ray_sample_kernel<8><<<grid_for(n * 8), kBlock, 0, s>>>(
                map->d, origins, directions, nears, fars, n, max_samples, grid2cell, counts,
                prefix, ray_indices, t_nears, t_fars, stage, stride);
    } else {
        ray_sample_kernel<1><<<grid_for(n), kBlock, 0, s>>>(
                map->d, origins, directions, nears, fars, n, max_samples, grid2cell, counts,
                prefix, ray_indices, t_nears, t_fars, stage, stride);
    }
    return 0;
}


int check_map(const ash_map* map) {
    if (map == nullptr) ASH_FAIL("null map handle");
    return 0;
}

// Whether a listing has entry i under index i: nothing has written to the heap
// since it was last 0, 1, 2, ... (no erase, no load) and no entry lives in the
// second region -- there is none, or the counters as the host knows them say
// that it is empty.
bool lists_in_index_order(const ash_map* map) {
    if (!heap_in_order(map)) return false;
    return !map->general_attached ||
           (map->counters_known && map->counters.general_live == 0);
}

int fill_buckets(ash_map* map, hipStream_t s) {
    const int64_t n16 = static_cast<int64_t>(map->d.nb) * kGroup;
    fill16_kernel<<<capped_grid(n16), kBlock, 0, s>>>(
            reinterpret_cast<uint4*>(map->d.buckets), n16, 0xFFFFFFFFu);
    ASH_LAUNCH_CHECK();
    map->table_stale = false;
    return 0;
}

// `lazy`: leave the bucket array to the next call that needs it (settle_table).
// `lazy` also leaves the key log while the heap is in its initial order.
int clear_table(ash_map* map, hipStream_t s, bool write_heap, int32_t size, bool lazy = false) {
    if (lazy) {
        map->table_stale = true;
    } else if (fill_buckets(map, s)) {
        return 1;
    }
    if (map->general_attached) {
        const int64_t g16 = static_cast<int64_t>(map->d.gslots) / 4;
        fill16_kernel<<<capped_grid(g16), kBlock, 0, s>>>(
                reinterpret_cast<uint4*>(map->d.gstate), g16, 0xFFFFFFFFu);
        ASH_LAUNCH_CHECK();
    }
    // The key log: every index is free again.  While nothing has written to the
    // heap since its last reset the indices in use are 0 .. size-1 and nothing
    // reads the log beyond the size: a lazy clear leaves the log alone and only
    // notes how far it holds entries (reset_heap_kernel); otherwise that part
    // of the log (read on the device, before the counters are reset below) is
    // emptied, or all of it once the heap has been written to.
    const bool keep_log = lazy && !map->heap_dirty;
    if (keep_log) {
        map->log_stale = true;
    } else {
        const int64_t n16 = (map->capacity + 1) / 2;
        // (a prefix of unknown length: few workgroups that loop, not one per
        // 4 KB of the capacity, most of which would start only to leave)
        empty_log_kernel<<<map->heap_dirty ? capped_grid(n16) : looping_grid(n16), kBlock, 0, s>>>(
                reinterpret_cast<uint4*>(map->d.klog), map->capacity, map->d.ctr,
                map->heap_dirty ? 0 : 1);
        ASH_LAUNCH_CHECK();
        map->log_stale = false;
    }
    // Inserts only read the heap; while nothing has written to it since the
    // last reset it still is 0, 1, 2, ... and only the counters are reset.
    const bool rewrite = write_heap && map->heap_dirty;
    int64_t span = rewrite && map->capacity > kNumCounters ? map->capacity : kNumCounters;
    reset_heap_kernel<<<grid_for(span), kBlock, 0, s>>>(
            map->d.heap, map->capacity, map->d.ctr, size, rewrite, keep_log);
    ASH_LAUNCH_CHECK();
    if (rewrite) map->heap_dirty = false;
    return 0;
}

}  // namespace

int give_up_heap_order(ash_map* map, hipStream_t s) {
    if (map->heap_dirty) return 0;
    map->heap_dirty = true;
    if (!map->log_stale) return 0;
    empty_log_tail_kernel<<<looping_grid(map->capacity), kBlock, 0, s>>>(
            map->d.klog, map->capacity, map->d.ctr);
    ASH_LAUNCH_CHECK();
    map->log_stale = false;
    return 0;
}

namespace {

template <int MODE>
int launch_insert(ash_map* map, const int32_t* keys, int64_t n,
                  const ValueArgs& va, int32_t* assigned, const int64_t* given,
                  hipStream_t s) {
    const unsigned g = grid_for(n, kHeapBlock);
    switch (map->key_dim) {
        case 1:
            insert_kernel<1, MODE><<<g, kHeapBlock, 0, s>>>(map->d, keys, n, va,
                                                        assigned, given);
            break;
        case 2:
            insert_kernel<2, MODE><<<g, kHeapBlock, 0, s>>>(map->d, keys, n, va,
                                                        assigned, given);
            break;
        case 3:
            insert_kernel<3, MODE><<<g, kHeapBlock, 0, s>>>(map->d, keys, n, va,
                                                        assigned, given);
            break;
        default:
            insert_kernel<4, MODE><<<g, kHeapBlock, 0, s>>>(map->d, keys, n, va,
                                                        assigned, given);
            break;
    }
    ASH_LAUNCH_CHECK();
    return 0;
}

template <int MODE>
int launch_selected(ash_map* map, bool codes, const int32_t* keys,
                    const int32_t* sel, const int32_t* nsel,
                    const ValueArgs& va, hipStream_t s) {
    // the selection is empty or short as a rule: a grid that costs little to
    // launch, whose workgroups stride over a long one
    constexpr unsigned g = 128;
    if (codes) {
        insert_selected_kernel<1, MODE, true>
                <<<g, kHeapBlock, 0, s>>>(map->d, keys, sel, nsel, va);
    } else {
        switch (map->key_dim) {
            case 1:
                insert_selected_kernel<1, MODE, false>
                        <<<g, kHeapBlock, 0, s>>>(map->d, keys, sel, nsel, va);
                break;
            case 2:
                insert_selected_kernel<2, MODE, false>
                        <<<g, kHeapBlock, 0, s>>>(map->d, keys, sel, nsel, va);
                break;
            case 3:
                insert_selected_kernel<3, MODE, false>
                        <<<g, kHeapBlock, 0, s>>>(map->d, keys, sel, nsel, va);
                break;
            default:
                insert_selected_kernel<4, MODE, false>
                        <<<g, kHeapBlock, 0, s>>>(map->d, keys, sel, nsel, va);
                break;
        }
    }
    ASH_LAUNCH_CHECK();
    return 0;
}

}  // namespace

// Every entry that reads or updates buckets calls this first.  The fill must
// not end up in a captured graph: replays would empty the table again.
int settle_table(ash_map* map, hipStream_t s) {
    if (!map->table_stale) return 0;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capturing) == hipSuccess &&
        capturing != hipStreamCaptureStatusNone) {
        ASH_FAIL("the table was cleared and not used since: run one call outside the capture first");
    }
    return fill_buckets(map, s);
}

void counters_changed(ash_map* map, bool inserted, hipStream_t s) {
    if (is_capturing(s)) map->replayed = true;
    map->counters_known = false;
    map->late_pending = false;   // what a queued read-back brings is out of date
    if (inserted) {
        ++map->unread_inserts;
    } else {
        map->maybe_tombstones = true;
    }
}

int check_batch(const ash_map* map, const void* keys, int64_t n) {
    if (check_map(map)) return 1;
    if (n < 0) ASH_FAIL("negative key count");
    if (n > 0 && keys == nullptr) ASH_FAIL("null keys pointer");
    if (n > (int64_t{1} << 31) - kHeapBlock) ASH_FAIL("too many keys in one call");
    return 0;
}

int erase_selected(ash_map* map, bool codes, const void* keys, const int32_t* sel,
                   const int32_t* nsel, hipStream_t s) {
    const int32_t* k = static_cast<const int32_t*>(keys);
    constexpr unsigned g = 64;   // the selection is empty or short as a rule
    if (codes) {
        erase_selected_kernel<1, true><<<g, kEraseBlock, 0, s>>>(map->d, k, sel, nsel);
    } else {
        switch (map->key_dim) {
            case 1:
                erase_selected_kernel<1, false><<<g, kEraseBlock, 0, s>>>(map->d, k, sel, nsel);
                break;
            case 2:
                erase_selected_kernel<2, false><<<g, kEraseBlock, 0, s>>>(map->d, k, sel, nsel);
                break;
            case 3:
                erase_selected_kernel<3, false><<<g, kEraseBlock, 0, s>>>(map->d, k, sel, nsel);
                break;
            default:
                erase_selected_kernel<4, false><<<g, kEraseBlock, 0, s>>>(map->d, k, sel, nsel);
                break;
        }
    }
    ASH_LAUNCH_CHECK();
    return 0;
}

int insert_selected(ash_map* map, bool codes, const void* keys,
                    const int32_t* sel, const int32_t* nsel,
                    const ValueArgs& va, hipStream_t s) {
    const int32_t* k = static_cast<const int32_t*>(keys);
    if (va.n > 0) {
        return launch_selected<kInsertFused>(map, codes, k, sel, nsel, va, s);
    }
    return launch_selected<kInsertKeys>(map, codes, k, sel, nsel, va, s);
}

}  // namespace ash

using namespace ash;

extern "C" {

const char* ash_last_error(void) { return g_last_error.c_str(); }

int ash_abi_version(void) { return 1; }

// The build passes the fingerprint of the kernel sources it compiles
// (torch-ash_amd/build.py: source_fingerprint).
#ifndef ASH_SOURCE_FINGERPRINT
#define ASH_SOURCE_FINGERPRINT "unknown"
#endif
const char* ash_source_fingerprint(void) { return ASH_SOURCE_FINGERPRINT; }

int ash_map_workspace_bytes(int key_dim, int64_t capacity, int64_t* table_bytes,
                            int64_t* general_bytes) {
    if (key_dim < 1 || key_dim > 4) ASH_FAIL("key_dim must be in 1..4");
    if (capacity < 1 || capacity > 0x7FFFFFF0ll) {
        ASH_FAIL("capacity must be in 1..2^31-16");
    }
    if (table_bytes) *table_bytes = table_workspace_bytes(capacity);
    if (general_bytes) *general_bytes = general_slots(capacity) * 20;
    return 0;
}

int ash_map_create(int key_dim, int64_t capacity, int32_t* heap, void* table_ws,
                   int64_t table_bytes, int device, void* stream,
                   ash_map_t** out) {
    if (out == nullptr) ASH_FAIL("null output handle");
    *out = nullptr;
    int64_t need = 0;
    if (ash_map_workspace_bytes(key_dim, capacity, &need, nullptr)) return 1;
    if (heap == nullptr || table_ws == nullptr) ASH_FAIL("null device buffer");
    if (table_bytes < need) ASH_FAIL("table workspace too small");
    if (reinterpret_cast<uintptr_t>(table_ws) % 256 != 0) {
        ASH_FAIL("table workspace must be 256-byte aligned");
    }
    DeviceGuard guard;
    ASH_HIP(guard.enter(device));
    ash_map* map = new ash_map();
    map->key_dim = key_dim;
    map->capacity = capacity;
    map->device = device;
    map->table_bytes = table_bytes;
    map->general_attached = false;
    map->table_stale = false;
    map->heap_dirty = true;   // the caller's buffer holds anything
    map->log_stale = false;
    map->staging = nullptr;
    map->early_event = map->late_event = nullptr;
    map->late_in_flight = map->late_pending = false;
    map->counters_known = true;   // a new map is empty and every counter is zero
    map->counters = {};
    map->maybe_tombstones = false;
    map->unread_inserts = 0;
    map->replayed = false;
    map->d.ctr = static_cast<int32_t*>(table_ws);
    map->d.buckets = reinterpret_cast<uint64_t*>(static_cast<char*>(table_ws) +
                                                 kHeaderBytes);
    map->d.klog = reinterpret_cast<uint64_t*>(static_cast<char*>(table_ws) +
                                              klog_offset(capacity));
    map->d.heap = heap;
    map->d.gstate = nullptr;
    map->d.gkeys = nullptr;
    map->d.nb = static_cast<uint32_t>(num_buckets(capacity));
    map->d.gslots = 0;
    map->d.capacity = static_cast<int32_t>(capacity);
    // (the fill of the bucket array is left to the first call that needs it: a
    // streaming insert, which writes every bucket itself, does not)
    if (clear_table(map, static_cast<hipStream_t>(stream), true, 0, true)) {
        delete map;
        return 1;
    }
    *out = map;
    return 0;
}

int ash_map_attach_general(ash_map_t* map, void* general_ws,
                           int64_t general_bytes, void* stream) {
    if (check_map(map)) return 1;
    if (map->general_attached) ASH_FAIL("general region already attached");
    if (general_ws == nullptr || general_bytes < kMinGeneralSlots * 20) {
        ASH_FAIL("general workspace too small");
    }
    // the largest power of two of slots that fits, up to what `capacity` keys need
    int64_t slots = kMinGeneralSlots;
    while (slots < general_slots(map->capacity) && slots * 2 * 20 <= general_bytes) slots <<= 1;
    if (reinterpret_cast<uintptr_t>(general_ws) % 256 != 0) {
        ASH_FAIL("general workspace must be 256-byte aligned");
    }
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    hipStream_t s = static_cast<hipStream_t>(stream);
    // keys first (16 B per slot, keeps them 16-byte aligned), then states
    map->d.gkeys = static_cast<int32_t*>(general_ws);
    map->d.gstate = map->d.gkeys + slots * 4;
    map->d.gslots = static_cast<uint32_t>(slots);
    map->general_attached = true;
    fill16_kernel<<<capped_grid(slots / 4), kBlock, 0, s>>>(
            reinterpret_cast<uint4*>(map->d.gstate), slots / 4, 0xFFFFFFFFu);
    ASH_LAUNCH_CHECK();
    set_counter_kernel<<<1, 64, 0, s>>>(map->d.ctr, kCtrExotic, 0);
    ASH_LAUNCH_CHECK();
    if (map->counters_known) map->counters.exotic_pending = 0;
    map->late_pending = false;
    return 0;
}

int ash_map_destroy(ash_map_t* map) {
    if (map == nullptr) return 0;
    // the device may still owe a write into the caller's page-locked landing
    // place; it must have arrived before the caller gives that memory back
    if (map->late_in_flight && map->late_event != nullptr) (void)hipEventSynchronize(map->late_event);
    if (map->early_event != nullptr) (void)hipEventDestroy(map->early_event);
    if (map->late_event != nullptr) (void)hipEventDestroy(map->late_event);
    delete map;
    return 0;
}

int ash_map_find(ash_map_t* map, const int32_t* keys, int64_t n,
                 int64_t* indices, uint8_t* masks, void* stream) {
    if (check_batch(map, keys, n)) return 1;
    if (n == 0) return 0;
    if (indices == nullptr || masks == nullptr) ASH_FAIL("null output pointer");
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (settle_table(map, s)) return 1;
    const unsigned g = grid_for(n);
    switch (map->key_dim) {
        case 1:
            find_kernel<1><<<g, kBlock, 0, s>>>(map->d, keys, n, indices, masks);
            break;
        case 2:
            find_kernel<2><<<g, kBlock, 0, s>>>(map->d, keys, n, indices, masks);
            break;
        case 3:
            find_kernel<3><<<g, kBlock, 0, s>>>(map->d, keys, n, indices, masks);
            break;
        default:
            find_kernel<4><<<g, kBlock, 0, s>>>(map->d, keys, n, indices, masks);
            break;
    }
    ASH_LAUNCH_CHECK();
    return 0;
}

int ash_grid_query(ash_map_t* map, const float* x, int64_t n, int grid_dim,
                   int64_t* grid_indices, int64_t* cell_indices, float* offsets,
                   uint8_t* masks, void* stream) {
    if (check_batch(map, x, n)) return 1;
    if (map->key_dim != 3) ASH_FAIL("grid queries need a map with 3-d keys");
    if (grid_dim < 1 || grid_dim > 1024) ASH_FAIL("grid_dim must be in 1..1024");
    if (n == 0) return 0;
    if (grid_indices == nullptr || cell_indices == nullptr ||
        offsets == nullptr || masks == nullptr) {
        ASH_FAIL("null output pointer");
    }
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    if (settle_table(map, static_cast<hipStream_t>(stream))) return 1;
    grid_query_kernel<<<grid_for(n), kBlock, 0,
                        static_cast<hipStream_t>(stream)>>>(
            map->d, x, n, static_cast<float>(grid_dim), grid_dim, grid_indices,
            cell_indices, offsets, masks);
    ASH_LAUNCH_CHECK();
    return 0;
}

namespace {

// Argument checks shared by the two activation entry points; `heads` is
// checked by the caller.
int check_activate(ash_map_t* map, const float* cells, int64_t n, int grid_dim,
                   int dilation, int bound_lo, int bound_hi, const uint8_t* touched,
                   const int32_t* coords) {
    if (check_batch(map, cells, n)) return 1;
    if (map->key_dim != 3) ASH_FAIL("block activation needs a map with 3-d keys");
    if (grid_dim < 1 || grid_dim > 1024) ASH_FAIL("grid_dim must be in 1..1024");
    if (dilation < 0 || dilation > 8) ASH_FAIL("dilation must be in 0..8");
    if (bound_lo > bound_hi) ASH_FAIL("empty block bounds");
    if (n > 0 && (touched == nullptr || coords == nullptr)) {
        ASH_FAIL("null output or scratch pointer");
    }
    return 0;
}

// The launches of an activation; the map's device is current, `heads` points
// to 64 + 3 n int32 of device memory.
int launch_activate(ash_map_t* map, const float* cells, int64_t n, int grid_dim,
                    int dilation, int bidirectional, int bound_lo, int bound_hi,
                    uint8_t* touched, int32_t* coords, int32_t* heads, hipStream_t s) {
    if (settle_table(map, s)) return 1;
    counters_changed(map, true, s);
    const int lo = bidirectional ? -dilation : 0;
    const int width = dilation - lo + 1;
    const float g = static_cast<float>(grid_dim);
    set_counter_kernel<<<1, 64, 0, s>>>(heads, 0, 0);
    ASH_LAUNCH_CHECK();
    activate_heads_kernel<<<grid_for(n, kHeadsBlock), kHeadsBlock, 0, s>>>(
            cells, n, g, bound_lo, bound_hi, heads);
    ASH_LAUNCH_CHECK();
    int64_t blocks = (n * width * width * width + kHeapBlock - 1) / kHeapBlock;
    if (blocks > 2048) blocks = 2048;
    const unsigned gb = static_cast<unsigned>(blocks);
    activate_kernel<false><<<gb, kHeapBlock, 0, s>>>(
            map->d, heads, lo, width, bound_lo, bound_hi, touched, coords);
    ASH_LAUNCH_CHECK();
    activate_kernel<true><<<gb, kHeapBlock, 0, s>>>(
            map->d, heads, lo, width, bound_lo, bound_hi, touched, coords);
    ASH_LAUNCH_CHECK();
    return 0;
}

// Address of `scratch` on each device, asked for once per device with that
// device current (every device holds its own copy at its own address).
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
int32_t* g_scratch_ptr[kMaxDevices] = {};

int scratch_on_current_device(int device, int32_t** out) {
    if (device < 0 || device >= kMaxDevices) ASH_FAIL("device number out of range");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[device] == nullptr) {
        void* p = nullptr;
        ASH_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (p == nullptr) ASH_FAIL("hipGetSymbolAddress returned no address for the scratch array");
        g_scratch_ptr[device] = static_cast<int32_t*>(p);
    }
    *out = g_scratch_ptr[device];
    return 0;
}

}  // namespace

int ash_grid_activate(ash_map_t* map, const float* cells, int64_t n,
                      int grid_dim, int dilation, int bidirectional,
                      int bound_lo, int bound_hi, uint8_t* touched,
                      int32_t* coords, int32_t* heads_scratch, void* stream) {
    if (check_activate(map, cells, n, grid_dim, dilation, bound_lo, bound_hi, touched, coords)) {
        return 1;
    }
    if (n == 0) return 0;
    if (heads_scratch == nullptr) ASH_FAIL("null output or scratch pointer");
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    return launch_activate(map, cells, n, grid_dim, dilation, bidirectional, bound_lo, bound_hi,
                           touched, coords, heads_scratch, static_cast<hipStream_t>(stream));
}

int ash_grid_activate_static(ash_map_t* map, const float* cells, int64_t n,
                             int grid_dim, int dilation, int bidirectional,
                             int bound_lo, int bound_hi, uint8_t* touched,
                             int32_t* coords, void* stream) {
    if (check_activate(map, cells, n, grid_dim, dilation, bound_lo, bound_hi, touched, coords)) {
        return 1;
    }
    if (n > kActivateStaticMax) {
        ASH_FAIL("ash_grid_activate_static takes at most " +
                 std::to_string(kActivateStaticMax) +
                 " positions per call (ASH_ACTIVATE_STATIC_MAX_POSITIONS); use "
                 "ash_grid_activate with a scratch buffer of the caller's for more");
    }
    if (n == 0) return 0;
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    int32_t* heads = nullptr;
    if (scratch_on_current_device(map->device, &heads)) return 1;
    return launch_activate(map, cells, n, grid_dim, dilation, bidirectional, bound_lo, bound_hi,
                           touched, coords, heads, static_cast<hipStream_t>(stream));
}

int ash_grid_activate_positions(ash_map_t* map, const float* positions, int64_t n,
                                const float* origin, float cell_size, int grid_dim,
                                int dilation, int bidirectional, int bound_lo, int bound_hi,
                                uint8_t* touched, int32_t* coords, void* stream) {
    if (check_activate(map, positions, n, grid_dim, dilation, bound_lo, bound_hi, touched,
                       coords)) {
        return 1;
    }
    if (!(cell_size > 0.f) || !(cell_size < INFINITY)) ASH_FAIL("cell_size must be positive and finite");
    if (n == 0) return 0;
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (settle_table(map, s)) return 1;
    counters_changed(map, true, s);
    RunsArgs a;
    a.x = positions;
    a.origin = origin;
    a.inv_cell = 1.0f / cell_size;
    a.g = static_cast<float>(grid_dim);
    a.n = n;
    a.off_lo = bidirectional ? -dilation : 0;
    a.width = dilation - a.off_lo + 1;
    a.bound_lo = bound_lo;
    a.bound_hi = bound_hi;
    const int64_t groups = (n + kRunPositions - 1) / kRunPositions;
    if (groups > 0x7FFFFFFFll) ASH_FAIL("too many positions in one call");
    activate_runs_kernel<<<static_cast<unsigned>(groups), kHeapBlock, 0, s>>>(
            map->d, a, touched, coords);
    ASH_LAUNCH_CHECK();
    return 0;
}

int ash_ray_find_near_far(ash_map_t* map, const float* ray_origins,
                          const float* ray_directions, const float* bbox_min,
                          const float* bbox_max, int64_t n, float t_min,
                          float t_max, float t_step, float grid2cell_multiplier,
                          float* ray_nears, float* ray_fars, void* stream) {
    (void)t_step;  // unused by the reference as well (ash/src/sampler.cu:21)
    if (check_batch(map, ray_origins, n)) return 1;
    if (map->key_dim != 3) {
        ASH_FAIL("hashmap is not a GPU hashmap of type <int, 3>, ray sample not supported");
    }
    if (!(grid2cell_multiplier > 0.f)) ASH_FAIL("grid2cell_multiplier must be positive");
    if (n == 0) return 0;
    if (ray_directions == nullptr || bbox_min == nullptr || bbox_max == nullptr ||
        ray_nears == nullptr || ray_fars == nullptr) {
        ASH_FAIL("null pointer in ray_find_near_far");
    }
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    if (settle_table(map, static_cast<hipStream_t>(stream))) return 1;
    // every step must advance t (else the march never ends), and their number
    // must stay finite
    const float half_block = static_cast<float>(grid2cell_multiplier * 0.5);
    if (t_min < t_max) {
        if (!(t_max + half_block > t_max) ||
            !((static_cast<double>(t_max) - t_min) / half_block < 1e8)) {
            ASH_FAIL("ray_find_near_far: the step is too small for this range");
        }
    }
    ray_near_far_kernel<<<grid_for(n, kBlock / 64), kBlock, 0, static_cast<hipStream_t>(stream)>>>(
            map->d, ray_origins, ray_directions, bbox_min, bbox_max, n, t_min,
            t_max, grid2cell_multiplier, ray_nears, ray_fars);
    ASH_LAUNCH_CHECK();
    return 0;
}

int ash_ray_sample(ash_map_t* map, const float* ray_origins,
                   const float* ray_directions, const float* ray_nears,
                   const float* ray_fars, int64_t n, int64_t max_samples_per_ray,
                   float grid2cell_multiplier, int64_t* counts,
                   const int64_t* prefix, int64_t* ray_indices, float* t_nears,
                   float* t_fars, void* stream) {
    if (check_batch(map, ray_origins, n)) return 1;
    if (map->key_dim != 3) {
        ASH_FAIL("hashmap is not a GPU hashmap of type <int, 3>, ray sample not supported");
    }
    if (!(grid2cell_multiplier > 0.f)) ASH_FAIL("grid2cell_multiplier must be positive");
    if (max_samples_per_ray < 1) ASH_FAIL("max_samples_per_ray must be positive");
    if (n == 0) return 0;
    if (ray_directions == nullptr || ray_nears == nullptr || ray_fars == nullptr) {
        ASH_FAIL("null pointer in ray_sample");
    }
    const bool assign = prefix != nullptr && ray_indices != nullptr &&
                        t_nears != nullptr && t_fars != nullptr;
    if ((counts != nullptr) == assign) {
        ASH_FAIL("ray_sample: pass either counts (allocation pass) or prefix and "
                 "the three outputs (assignment pass)");
    }
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    if (settle_table(map, static_cast<hipStream_t>(stream))) return 1;
    launch_ray_sample(map, ray_origins, ray_directions, ray_nears, ray_fars, n,
                      static_cast<float>(max_samples_per_ray), grid2cell_multiplier, counts,
                      prefix, ray_indices, t_nears, t_fars, nullptr, 0,
                      static_cast<hipStream_t>(stream));
    ASH_LAUNCH_CHECK();
    return 0;
}

int ash_ray_sample_staged(ash_map_t* map, const float* ray_origins,
                          const float* ray_directions, const float* ray_nears,
                          const float* ray_fars, int64_t n, int64_t max_samples_per_ray,
                          float grid2cell_multiplier, int64_t* counts, float* stage,
                          int64_t stride, void* stream) {
    if (check_batch(map, ray_origins, n)) return 1;
    if (map->key_dim != 3) {
        ASH_FAIL("hashmap is not a GPU hashmap of type <int, 3>, ray sample not supported");
    }
    if (!(grid2cell_multiplier > 0.f)) ASH_FAIL("grid2cell_multiplier must be positive");
    if (max_samples_per_ray < 1) ASH_FAIL("max_samples_per_ray must be positive");
    if (stride < 1) ASH_FAIL("ray_sample_staged: stride must be positive");
    if (n == 0) return 0;
    if (ray_directions == nullptr || ray_nears == nullptr || ray_fars == nullptr ||
        counts == nullptr || stage == nullptr) {
        ASH_FAIL("null pointer in ray_sample_staged");
    }
    if (reinterpret_cast<uintptr_t>(stage) % 8 != 0) ASH_FAIL("ray_sample_staged: stage must be 8-byte aligned");
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    if (settle_table(map, static_cast<hipStream_t>(stream))) return 1;
    launch_ray_sample(map, ray_origins, ray_directions, ray_nears, ray_fars, n,
                      static_cast<float>(max_samples_per_ray), grid2cell_multiplier, counts,
                      nullptr, nullptr, nullptr, nullptr, reinterpret_cast<float2*>(stage),
                      stride, static_cast<hipStream_t>(stream));
    ASH_LAUNCH_CHECK();
    return 0;
}

int ash_ray_sample_compact(const int64_t* counts, const int64_t* prefix, const float* stage,
                           int64_t stride, int64_t n, int64_t* ray_indices, float* t_nears,
                           float* t_fars, void* stream) {
    if (n < 0 || stride < 1) ASH_FAIL("ray_sample_compact: bad sizes");
    if (n == 0) return 0;
    if (counts == nullptr || prefix == nullptr || stage == nullptr || ray_indices == nullptr ||
        t_nears == nullptr || t_fars == nullptr) {
        ASH_FAIL("null pointer in ray_sample_compact");
    }
    if (n > ((int64_t{1} << 32) - kBlock) / stride) ASH_FAIL("ray_sample_compact: too many slots");
    ray_compact_kernel<<<grid_for(n * stride), kBlock, 0, static_cast<hipStream_t>(stream)>>>(
            counts, prefix, reinterpret_cast<const float2*>(stage), stride, n, ray_indices,
            t_nears, t_fars);
    ASH_LAUNCH_CHECK();
    return 0;
}

int ash_map_insert_keys(ash_map_t* map, const int32_t* keys, int64_t n,
                        void* stream) {
    if (check_batch(map, keys, n)) return 1;
    if (n == 0) return 0;
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    if (settle_table(map, static_cast<hipStream_t>(stream))) return 1;
    counters_changed(map, true, static_cast<hipStream_t>(stream));
    ValueArgs va = {};
    return launch_insert<kInsertKeys>(map, keys, n, va, nullptr, nullptr,
                                      static_cast<hipStream_t>(stream));
}

int ash_map_insert_needs_scratch(int n_values, const int64_t* row_bytes) {
    if (n_values <= 0) return 0;
    if (n_values > kMaxFusedValues) return 1;
    for (int v = 0; v < n_values; ++v) {
        if (row_bytes[v] % 4 != 0 || row_bytes[v] > kMaxFusedRowDwords * 4) {
            return 1;
        }
    }
    return 0;
}

int ash_scatter_rows(const void* src, void* dst, const int32_t* assigned,
                     int64_t n, int64_t row_bytes, void* stream) {
    if (n == 0 || row_bytes == 0) return 0;
    if (src == nullptr || dst == nullptr || assigned == nullptr) {
        ASH_FAIL("null pointer in scatter");
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uintptr_t align = reinterpret_cast<uintptr_t>(src) |
                            reinterpret_cast<uintptr_t>(dst) |
                            static_cast<uintptr_t>(row_bytes);
    if (align % 16 == 0) {
        const int64_t upr = row_bytes / 16;
        scatter_rows_kernel<uint4><<<looping_grid(n * upr), kBlock, 0, s>>>(
                static_cast<const uint4*>(src), static_cast<uint4*>(dst),
                assigned, n, upr);
    } else if (align % 4 == 0) {
        const int64_t upr = row_bytes / 4;
        scatter_rows_kernel<uint32_t><<<looping_grid(n * upr), kBlock, 0, s>>>(
                static_cast<const uint32_t*>(src), static_cast<uint32_t*>(dst),
                assigned, n, upr);
    } else {
        scatter_rows_kernel<uint8_t><<<looping_grid(n * row_bytes), kBlock, 0,
                                       s>>>(static_cast<const uint8_t*>(src),
                                            static_cast<uint8_t*>(dst),
                                            assigned, n, row_bytes);
    }
    ASH_LAUNCH_CHECK();
    return 0;
}

int ash_gather_rows(int n_values, const void* const* src, void* const* dst,
                    const int64_t* row_bytes, const int64_t* src_rows,
                    const int64_t* indices, int64_t n, void* stream) {
    if (n_values < 1 || n_values > kMaxFusedValues) {
        ASH_FAIL("gather_rows takes 1.." + std::to_string(kMaxFusedValues) + " tensors per call");
    }
    if (n < 0) ASH_FAIL("negative row count");
    if (src == nullptr || dst == nullptr || row_bytes == nullptr || src_rows == nullptr) {
        ASH_FAIL("null value tables");
    }
    if (n == 0) return 0;
    GatherArgs a = {};
    a.n = n_values;
    int64_t most = 0;
    for (int v = 0; v < n_values; ++v) {
        if (src[v] == nullptr || dst[v] == nullptr) ASH_FAIL("null value tensor");
        if (row_bytes[v] <= 0 || row_bytes[v] % 4 != 0) {
            ASH_FAIL("gather_rows: rows must be a positive multiple of 4 bytes");
        }
        if (src_rows[v] < 0) ASH_FAIL("negative source row count");
        a.src[v] = static_cast<const uint32_t*>(src[v]);
        a.dst[v] = static_cast<uint32_t*>(dst[v]);
        a.row_dwords[v] = static_cast<int32_t>(row_bytes[v] / 4);
        a.src_rows[v] = src_rows[v];
        const int64_t words = n * a.row_dwords[v];
        most = words > most ? words : most;
    }
    PointerGuard guard;
    ASH_HIP(guard.enter_for(src[0]));
    if (indices == nullptr) {
        int64_t g = (most / 4 + kBlock - 1) / kBlock;
        if (g > 256 * 64) g = 256 * 64;
        if (g < 1) g = 1;
        copy_first_rows_kernel<<<static_cast<unsigned>(g), kBlock, 0,
                                 static_cast<hipStream_t>(stream)>>>(a, n);
        ASH_LAUNCH_CHECK();
        return 0;
    }
    gather_rows_kernel<<<looping_grid(most), kBlock, 0, static_cast<hipStream_t>(stream)>>>(
            a, indices, n);
    ASH_LAUNCH_CHECK();
    return 0;
}

int ash_map_insert(ash_map_t* map, const int32_t* keys, int64_t n, int n_values,
                   const void* const* src, void* const* dst,
                   const int64_t* row_bytes, int32_t* assigned, void* stream) {
    if (check_batch(map, keys, n)) return 1;
    if (n_values < 0) ASH_FAIL("negative value count");
    if (n_values == 0) return ash_map_insert_keys(map, keys, n, stream);
    if (src == nullptr || dst == nullptr || row_bytes == nullptr) {
        ASH_FAIL("null value tables");
    }
    for (int v = 0; v < n_values; ++v) {
        if (src[v] == nullptr || dst[v] == nullptr) ASH_FAIL("null value tensor");
        if (row_bytes[v] <= 0) ASH_FAIL("value rows must not be empty");
    }
    if (n == 0) return 0;
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (settle_table(map, s)) return 1;
    counters_changed(map, true, s);
    ValueArgs va = {};
    if (!ash_map_insert_needs_scratch(n_values, row_bytes)) {
        va.n = n_values;
        for (int v = 0; v < n_values; ++v) {
            va.src[v] = static_cast<const uint32_t*>(src[v]);
            va.dst[v] = static_cast<uint32_t*>(dst[v]);
            va.row_dwords[v] = static_cast<int32_t>(row_bytes[v] / 4);
        }
        return launch_insert<kInsertFused>(map, keys, n, va, nullptr, nullptr,
                                           s);
    }
    if (assigned == nullptr) {
        ASH_FAIL("these value rows need the `assigned` temporary");
    }
    if (launch_insert<kInsertAssign>(map, keys, n, va, assigned, nullptr, s)) {
        return 1;
    }
    for (int v = 0; v < n_values; ++v) {
        if (ash_scatter_rows(src[v], dst[v], assigned, n, row_bytes[v], stream)) {
            return 1;
        }
    }
    return 0;
}

int ash_map_erase(ash_map_t* map, const int32_t* keys, int64_t n,
                  void* stream) {
    if (check_batch(map, keys, n)) return 1;
    if (n == 0) return 0;
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (settle_table(map, s)) return 1;
    if (give_up_heap_order(map, s)) return 1;   // freed indices go back onto the heap
    counters_changed(map, false, s);
    const unsigned g = grid_for(n, kEraseBlock);
    switch (map->key_dim) {
        case 1:
            erase_kernel<1><<<g, kEraseBlock, 0, s>>>(map->d, keys, n);
            break;
        case 2:
            erase_kernel<2><<<g, kEraseBlock, 0, s>>>(map->d, keys, n);
            break;
        case 3:
            erase_kernel<3><<<g, kEraseBlock, 0, s>>>(map->d, keys, n);
            break;
        default:
            erase_kernel<4><<<g, kEraseBlock, 0, s>>>(map->d, keys, n);
            break;
    }
    ASH_LAUNCH_CHECK();
    return 0;
}

int ash_map_clear(ash_map_t* map, void* stream) {
    if (check_map(map)) return 1;
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (is_capturing(s)) map->replayed = true;
    if (map->replayed) {
        // what replays leave behind is unknown: everything is cleared now
        if (settle_table(map, s)) return 1;
        map->heap_dirty = true;
        if (clear_table(map, s, true, 0, false)) return 1;
        map->heap_dirty = true;   // (whatever the flag would say: see heap_in_order)
    } else if (clear_table(map, s, true, 0, true)) {
        return 1;
    }
    // every counter is zero again: known without a read-back
    map->counters_known = true;
    map->counters = {};
    map->late_pending = false;
    map->maybe_tombstones = false;
    map->unread_inserts = 0;
    return 0;
}

namespace {

void decode_counters(const int32_t* host, ash_counters& c) {
    c.size = host[kCtrSize];
    c.dropped = host[kCtrDropped];
    c.tombstones = host[kCtrTombs];
    c.exotic_pending = host[kCtrExotic];
    c.load_refused = host[kCtrLoadDup];
    c.touched = host[kCtrTouched];
    c.general_live = host[kCtrGenLive];
    c.general_tombstones = host[kCtrGenTombs];
}

int ensure_events(ash_map* map) {
    if (map->early_event == nullptr) {
        ASH_HIP(hipEventCreateWithFlags(&map->early_event, hipEventDisableTiming));
    }
    if (map->late_event == nullptr) {
        ASH_HIP(hipEventCreateWithFlags(&map->late_event, hipEventDisableTiming));
    }
    return 0;
}

// A copy into the map's own landing place that may still be under way has to
// arrive before that memory is written or read for something else.
int settle_landing_place(ash_map* map) {
    if (map->late_in_flight) {
        ASH_HIP(hipEventSynchronize(map->late_event));
        map->late_in_flight = false;
    }
    return 0;
}

// Brings map->counters up to date (the map's device is current): they are
// known already, or a read-back queued behind the latest insert brings them,
// or they are copied now, which waits for `s`.  `staging`: eight int32 of
// page-locked host memory of the calling thread's, or null -- a copy into
// pageable memory goes through the runtime's own staging and takes about twice
// as long (25 against 13 us on an idle device).
int refresh_counters(ash_map* map, int32_t* staging, hipStream_t s) {
    if (map->replayed) {
        if (settle_landing_place(map)) return 1;
        map->counters_known = map->late_pending = false;
    }
    if (map->counters_known) return 0;
    if (map->late_pending) {
        if (settle_landing_place(map)) return 1;
        map->late_pending = false;
        decode_counters(map->staging, map->counters);
    } else {
        if (is_capturing(s)) {
            ASH_FAIL("the table's counters cannot be read while the stream is being captured");
        }
        int32_t pageable[kHostCounters] = {0};
        int32_t* host = staging != nullptr ? staging : pageable;
        ASH_HIP(hipMemcpyAsync(host, map->d.ctr, sizeof(pageable), hipMemcpyDeviceToHost, s));
        ASH_HIP(hipStreamSynchronize(s));
        decode_counters(host, map->counters);
    }
    map->counters_known = true;
    map->unread_inserts = 0;
    if (map->counters.dropped > 0 || map->counters.tombstones > 0) map->maybe_tombstones = true;
    return 0;
}

// Inserts whose counters nobody read (deferred activations) between two looks
// at them for tombstone upkeep.
constexpr int kUpkeepEvery = 64;

int64_t rebuild_scratch_bytes(const ash_map* map) {
    const int64_t keys = (map->capacity * map->key_dim * 4 + 255) & ~int64_t{255};
    return keys + map->capacity * 8;
}

// keep at least a fifth of the slots truly empty -- of the bucket array, and
// of the second region on its own account (`general_used`: its entries and
// tombstones; it may be much smaller than the table)
bool should_rebuild(const ash_map* map, int64_t size, int64_t tombstones, int64_t incoming,
                    int64_t general_used = 0, int64_t general_tombstones = 0) {
    if (tombstones <= 0) return false;
    int64_t room = map->capacity - size;
    if (room < 0) room = 0;
    const int64_t arriving = incoming < room ? incoming : room;
    const int64_t slots = static_cast<int64_t>(map->d.nb) * kSlots;
    if ((size + tombstones + arriving) * 5 > slots * 4) return true;
    return map->general_attached && general_tombstones > 0 &&
           general_used * 5 > static_cast<int64_t>(map->d.gslots) * 4;
}

// Before an insert of `incoming` keys (the map's device is current, `s` is not
// being captured): if earlier erases or refused keys may have left
// tombstones, looks at the counters and re-places the live entries into an
// emptied table when too few empty slots would remain.
int upkeep(ash_map* map, int64_t incoming, void* scratch, int64_t scratch_bytes,
           int32_t* staging, hipStream_t s) {
    if (map->late_pending && refresh_counters(map, staging, s)) return 1;
    if (map->unread_inserts >= kUpkeepEvery || map->replayed) map->maybe_tombstones = true;
    if (!map->maybe_tombstones) return 0;
    if (refresh_counters(map, staging, s)) return 1;
    const ash_counters& c = map->counters;
    map->maybe_tombstones = c.tombstones > 0;
    if (!should_rebuild(map, c.size, c.tombstones, incoming,
                        c.general_live + c.general_tombstones, c.general_tombstones)) {
        return 0;
    }
    int32_t* keys = nullptr;
    int64_t* indices = nullptr;
    if (map->general_attached && c.size > 0) {
        // entries of the second region do not stand in the key log: the pairs
        // are listed into the caller's scratch and put back from there
        if (scratch == nullptr || scratch_bytes < rebuild_scratch_bytes(map)) {
            ASH_FAIL("scratch too small to re-place the entries: size it with "
                     "ash_map_insert_scratch_bytes before every insert");
        }
        keys = static_cast<int32_t*>(scratch);
        indices = reinterpret_cast<int64_t*>(
                static_cast<char*>(scratch) +
                ((map->capacity * map->key_dim * 4 + 255) & ~int64_t{255}));
    }
    if (ash_map_rebuild(map, keys, indices, c.size, s)) return 1;
    map->counters.tombstones = 0;
    map->counters_known = true;
    map->maybe_tombstones = false;
    return 0;
}

}  // namespace

int ash_map_set_staging(ash_map_t* map, int32_t* staging) {
    if (check_map(map)) return 1;
    if (settle_landing_place(map)) return 1;
    if (map->late_pending) {
        // what the old landing place holds is the latest state of the counters
        decode_counters(map->staging, map->counters);
        map->counters_known = true;
        map->late_pending = false;
    }
    map->staging = staging;
    return 0;
}

int ash_map_counters(ash_map_t* map, int32_t* staging, int64_t out[7], void* stream) {
    if (check_map(map)) return 1;
    if (out == nullptr) ASH_FAIL("null status output");
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    if (refresh_counters(map, staging, static_cast<hipStream_t>(stream))) return 1;
    const ash_counters& c = map->counters;
    out[0] = c.size;
    out[1] = c.dropped;
    out[2] = c.tombstones;
    out[3] = c.exotic_pending;
    out[4] = c.load_refused;
    out[5] = c.touched;
    out[6] = c.general_live;
    return 0;
}

int ash_map_counters_pending(ash_map_t* map) {
    return map != nullptr && map->late_pending ? 1 : 0;
}

int ash_map_known_size(ash_map_t* map, int64_t* size) {
    if (check_map(map)) return -1;
    if (size == nullptr) {
        set_error("null size output");
        return -1;
    }
    if (map->replayed) return 0;
    if (!map->counters_known) {
        if (!map->late_pending) return 0;
        DeviceGuard guard;
        if (guard.enter(map->device) != hipSuccess || refresh_counters(map, nullptr, nullptr)) {
            return -1;
        }
    }
    *size = map->counters.size;
    return 1;
}

int ash_map_status(ash_map_t* map, int64_t out[5], void* stream) {
    if (check_map(map)) return 1;
    if (out == nullptr) ASH_FAIL("null status output");
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    // always a copy from the device
    map->counters_known = false;
    map->late_pending = false;
    if (refresh_counters(map, nullptr, static_cast<hipStream_t>(stream))) return 1;
    const ash_counters& c = map->counters;
    out[0] = c.size;
    out[1] = c.dropped;
    out[2] = c.tombstones;
    out[3] = c.exotic_pending;
    out[4] = c.load_refused;
    return 0;
}

int ash_map_upkeep(ash_map_t* map, int64_t incoming, void* scratch, int64_t scratch_bytes,
                   int32_t* staging, void* stream) {
    if (check_map(map)) return 1;
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (is_capturing(s)) return 0;
    return upkeep(map, incoming, scratch, scratch_bytes, staging, s);
}

namespace {

// Which path an insert of this batch takes; *bytes = device scratch it needs.
enum { kPathPerKey = 0, kPathAssigned = 1, kPathStreaming = 2 };

int plan_insert(ash_map_t* map, int64_t n, int n_values, const int64_t* row_bytes, int policy,
                int* path, int64_t* bytes) {
    if (policy < ASH_STREAMING_AUTO || policy > ASH_STREAMING_NEVER) ASH_FAIL("unknown policy");
    if (n_values < 0) ASH_FAIL("negative value count");
    if (n_values > 0 && row_bytes == nullptr) ASH_FAIL("null value tables");
    *path = kPathPerKey;
    *bytes = 0;
    if (n_values > 0 && ash_map_insert_needs_scratch(n_values, row_bytes)) {
        *path = kPathAssigned;
        *bytes = n * 4;
    } else if (policy != ASH_STREAMING_NEVER) {
        int64_t ws = 0;
        int worthwhile = 0;
        if (ash_map_bulk_workspace_bytes(map, n, n_values, row_bytes, &ws, &worthwhile)) return 1;
        if (ws > 0 && (worthwhile || policy == ASH_STREAMING_ALWAYS)) {
            *path = kPathStreaming;
            *bytes = ws;
        }
    }
    // a map with a second region re-places its entries through the scratch
    if (map->general_attached &&
        (map->maybe_tombstones || map->unread_inserts >= kUpkeepEvery || map->replayed)) {
        const int64_t r = rebuild_scratch_bytes(map);
        if (r > *bytes) *bytes = r;
    }
    return 0;
}

}  // namespace

int ash_map_insert_scratch_bytes(ash_map_t* map, int64_t n, int n_values,
                                 const int64_t* row_bytes, int policy, int64_t* bytes) {
    if (check_map(map)) return 1;
    if (bytes == nullptr) ASH_FAIL("null output pointer");
    if (n < 0) ASH_FAIL("negative key count");
    int path = 0;
    return plan_insert(map, n, n_values, row_bytes, policy, &path, bytes);
}

int ash_map_insert_auto(ash_map_t* map, const int32_t* keys, int64_t n, int n_values,
                        const void* const* src, void* const* dst, const int64_t* row_bytes,
                        void* scratch, int64_t scratch_bytes, int policy, int32_t* staging,
                        void* stream) {
    if (check_batch(map, keys, n)) return 1;
    if (n == 0) return 0;
    int path = 0;
    int64_t need = 0;
    if (plan_insert(map, n, n_values, row_bytes, policy, &path, &need)) return 1;
    if (need > 0 && (scratch == nullptr || scratch_bytes < need)) {
        ASH_FAIL("insert scratch too small: size it with ash_map_insert_scratch_bytes");
    }
    if (need > 0 && reinterpret_cast<uintptr_t>(scratch) % 256 != 0) {
        ASH_FAIL("insert scratch must be 256-byte aligned");
    }
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool capturing = is_capturing(s);
    // (a capture replays launches only: no look at the counters, no upkeep;
    // refused keys stay in the counters for a later call to find)
    if (!capturing && upkeep(map, n, scratch, scratch_bytes, staging, s)) return 1;
    if (path == kPathStreaming) {
        int32_t* early = nullptr;
        if (!capturing && map->staging != nullptr) {
            if (ensure_events(map) || settle_landing_place(map)) return 1;
            early = map->staging + kHostCounters;
        }
        if (insert_bulk(map, keys, n, n_values, src, dst, row_bytes, scratch, scratch_bytes,
                        early, early != nullptr ? map->early_event : nullptr, stream)) {
            return 1;
        }
        if (capturing) return 0;
        if (early != nullptr) {
            // Only keys that the first pass hands to the per-key kernel can be
            // waiting for the second region; their number arrives a quarter
            // into the call's work.  None: the counters are fetched behind the
            // insert without waiting for them.
            ASH_HIP(hipEventSynchronize(map->early_event));
            if (*early == 0) {
                ASH_HIP(hipMemcpyAsync(map->staging, map->d.ctr, kHostCounters * sizeof(int32_t),
                                       hipMemcpyDeviceToHost, s));
                ASH_HIP(hipEventRecord(map->late_event, s));
                map->late_in_flight = true;
                map->late_pending = true;
                map->unread_inserts = 0;
                return 0;
            }
        }
    } else {
        if (ash_map_insert(map, keys, n, n_values, src, dst, row_bytes,
                           path == kPathAssigned ? static_cast<int32_t*>(scratch) : nullptr,
                           stream)) {
            return 1;
        }
        if (capturing) return 0;
    }
    if (refresh_counters(map, staging, s)) return 1;
    if (map->counters.exotic_pending > 0 && map->general_attached) {
        fold_waiting_keys_kernel<<<1, 64, 0, s>>>(map->d.ctr);
        ASH_LAUNCH_CHECK();
        map->counters.dropped += map->counters.exotic_pending;
        map->counters.exotic_pending = 0;
        map->maybe_tombstones = true;
    }
    if (map->counters.exotic_pending > 0) {
        set_error("keys that do not fit the packed code are waiting for the second region: "
                  "attach it (ash_map_attach_general) and issue the insert again");
        return ASH_NEEDS_GENERAL;
    }
    return 0;
}

int ash_map_erase_scratch_bytes(ash_map_t* map, int64_t n, int policy, int64_t* bytes) {
    if (check_map(map)) return 1;
    if (bytes == nullptr) ASH_FAIL("null output pointer");
    if (policy < ASH_STREAMING_AUTO || policy > ASH_STREAMING_NEVER) ASH_FAIL("unknown policy");
    *bytes = 0;
    if (policy == ASH_STREAMING_NEVER) return 0;
    int64_t ws = 0;
    int worthwhile = 0;
    if (ash_map_erase_bulk_query(map, n, &ws, &worthwhile)) return 1;
    if (ws > 0 && (worthwhile || policy == ASH_STREAMING_ALWAYS)) *bytes = ws;
    return 0;
}

int ash_map_erase_auto(ash_map_t* map, const int32_t* keys, int64_t n, void* scratch,
                       int64_t scratch_bytes, int policy, void* stream) {
    if (check_batch(map, keys, n)) return 1;
    if (n == 0) return 0;
    int64_t need = 0;
    if (ash_map_erase_scratch_bytes(map, n, policy, &need)) return 1;
    if (need == 0) return ash_map_erase(map, keys, n, stream);
    if (scratch == nullptr || scratch_bytes < need) {
        ASH_FAIL("erase scratch too small: size it with ash_map_erase_scratch_bytes");
    }
    return ash_map_erase_bulk(map, keys, n, scratch, scratch_bytes, stream);
}

int ash_grid_collect_touched(ash_map_t* map, uint8_t* touched, const int32_t* block_coords,
                             int64_t* out_indices, int32_t* out_coords, void* stream) {
    if (check_map(map)) return 1;
    if (touched == nullptr || block_coords == nullptr || out_indices == nullptr ||
        out_coords == nullptr) {
        ASH_FAIL("null pointer in grid_collect_touched");
    }
    if (map->capacity > kCollectMaxBlocks) ASH_FAIL("grid_collect_touched: more than ASH_COLLECT_MAX_BLOCKS rows");
    if (reinterpret_cast<uintptr_t>(touched) % 4 != 0) ASH_FAIL("grid_collect_touched: flags must be 4-byte aligned");
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    const int64_t per_group = int64_t{4} * kCollectThreads;   // flags of a one-word-per-thread chunk
    int64_t groups = (map->capacity + per_group - 1) / per_group;
    if (groups > kCollectGroups) groups = kCollectGroups;
    const int words = static_cast<int>((map->capacity + groups * per_group - 1) / (groups * per_group));
    groups = (map->capacity + words * per_group - 1) / (words * per_group);   // no empty chunks
    map->counters_known = false;   // the number of listed rows is one of them
    map->late_pending = false;
    collect_touched_kernel<<<static_cast<unsigned>(groups), kCollectThreads, 0,
                             static_cast<hipStream_t>(stream)>>>(
            touched, block_coords, map->capacity, words, out_indices, out_coords, map->d.ctr);
    ASH_LAUNCH_CHECK();
    return 0;
}

int ash_map_size(ash_map_t* map, int64_t* size, void* stream) {
    if (size == nullptr) ASH_FAIL("null size output");
    int64_t c[7];
    if (ash_map_counters(map, nullptr, c, stream)) return 1;
    *size = c[0];
    return 0;
}

int ash_map_items(ash_map_t* map, int32_t* keys_out, int64_t* indices_out,
                  int64_t n_expected, void* stream) {
    if (check_map(map)) return 1;
    if (n_expected < 0) ASH_FAIL("negative item count");
    if (n_expected == 0) return 0;
    if (keys_out == nullptr || indices_out == nullptr) {
        ASH_FAIL("null output pointer");
    }
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (settle_table(map, s)) return 1;
    const int identity = heap_in_order(map) ? 1 : 0;
    const bool none_in_general = !map->general_attached ||
                                 (map->counters_known && map->counters.general_live == 0);
    if (lists_in_index_order(map)) {
        const int64_t n = n_expected < map->capacity ? n_expected : map->capacity;
        const unsigned gd = grid_for(n);
        switch (map->key_dim) {
            case 1:
                items_dense_kernel<1><<<gd, kBlock, 0, s>>>(map->d, keys_out, indices_out, n);
                break;
            case 2:
                items_dense_kernel<2><<<gd, kBlock, 0, s>>>(map->d, keys_out, indices_out, n);
                break;
            case 3:
                items_dense_kernel<3><<<gd, kBlock, 0, s>>>(map->d, keys_out, indices_out, n);
                break;
            default:
                items_dense_kernel<4><<<gd, kBlock, 0, s>>>(map->d, keys_out, indices_out, n);
                break;
        }
        ASH_LAUNCH_CHECK();
        return 0;
    }
    set_counter_kernel<<<1, 64, 0, s>>>(map->d.ctr, kCtrCursor, 0);
    ASH_LAUNCH_CHECK();
    const unsigned g = grid_for(map->capacity, kItemsSpan);
    switch (map->key_dim) {
        case 1:
            items_kernel<1><<<g, kItemsBlock, 0, s>>>(map->d, keys_out, indices_out,
                                                 n_expected, identity);
            break;
        case 2:
            items_kernel<2><<<g, kItemsBlock, 0, s>>>(map->d, keys_out, indices_out,
                                                 n_expected, identity);
            break;
        case 3:
            items_kernel<3><<<g, kItemsBlock, 0, s>>>(map->d, keys_out, indices_out,
                                                 n_expected, identity);
            break;
        default:
            items_kernel<4><<<g, kItemsBlock, 0, s>>>(map->d, keys_out, indices_out,
                                                 n_expected, identity);
            break;
    }
    ASH_LAUNCH_CHECK();
    if (!none_in_general) {
        const unsigned gg = grid_for(map->d.gslots);
        switch (map->key_dim) {
            case 1:
                items_general_kernel<1><<<gg, kBlock, 0, s>>>(
                        map->d, keys_out, indices_out, n_expected);
                break;
            case 2:
                items_general_kernel<2><<<gg, kBlock, 0, s>>>(
                        map->d, keys_out, indices_out, n_expected);
                break;
            case 3:
                items_general_kernel<3><<<gg, kBlock, 0, s>>>(
                        map->d, keys_out, indices_out, n_expected);
                break;
            default:
                items_general_kernel<4><<<gg, kBlock, 0, s>>>(
                        map->d, keys_out, indices_out, n_expected);
                break;
        }
        ASH_LAUNCH_CHECK();
    }
    return 0;
}

int ash_map_should_rebuild(ash_map_t* map, int64_t size, int64_t tombstones,
                           int64_t incoming) {
    if (map == nullptr) return 0;
    return should_rebuild(map, size, tombstones, incoming) ? 1 : 0;
}

int ash_map_rebuild(ash_map_t* map, int32_t* keys_scratch,
                    int64_t* indices_scratch, int64_t n, void* stream) {
    if (check_map(map)) return 1;
    if (n < 0 || n > map->capacity) ASH_FAIL("rebuild: bad entry count");
    // Without a second region every entry stands in the key log under its
    // index and is put back from there; with one, the pairs are listed into the
    // caller's scratch first.
    const bool from_log = !map->general_attached;
    if (!from_log && n > 0 && (keys_scratch == nullptr || indices_scratch == nullptr)) {
        ASH_FAIL("rebuild: null scratch pointer");
    }
    if (!from_log && n > 0 && ash_map_items(map, keys_scratch, indices_scratch, n, stream)) {
        return 1;
    }
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (fill_buckets(map, s)) return 1;
    if (map->general_attached) {
        const int64_t g16 = static_cast<int64_t>(map->d.gslots) / 4;
        fill16_kernel<<<capped_grid(g16), kBlock, 0, s>>>(
                reinterpret_cast<uint4*>(map->d.gstate), g16, 0xFFFFFFFFu);
        ASH_LAUNCH_CHECK();
        set_counter_kernel<<<1, 64, 0, s>>>(map->d.ctr, kCtrGenLive, 0);   // counted again below
        ASH_LAUNCH_CHECK();
        set_counter_kernel<<<1, 64, 0, s>>>(map->d.ctr, kCtrGenTombs, 0);
        ASH_LAUNCH_CHECK();
    }
    set_counter_kernel<<<1, 64, 0, s>>>(map->d.ctr, kCtrTombs, 0);
    ASH_LAUNCH_CHECK();
    map->counters_known = false;
    map->late_pending = false;
    if (n == 0) return 0;
    if (from_log) {
        int64_t g = (map->capacity + kHeapBlock - 1) / kHeapBlock;
        if (g > 256 * 16) g = 256 * 16;
        replace_from_log_kernel<<<static_cast<unsigned>(g), kHeapBlock, 0, s>>>(
                map->d, heap_in_order(map) ? 1 : 0);
        ASH_LAUNCH_CHECK();
        return 0;
    }
    ValueArgs va = {};
    return launch_insert<kInsertLoad>(map, keys_scratch, n, va, nullptr,
                                      indices_scratch, s);
}

int ash_map_items_in_index_order(ash_map_t* map, int* dense) {
    if (check_map(map)) return 1;
    if (dense == nullptr) ASH_FAIL("null output pointer");
    *dense = lists_in_index_order(map) ? 1 : 0;
    return 0;
}

int ash_map_load(ash_map_t* map, const int32_t* keys, const int64_t* indices,
                 int64_t n, const int32_t* heap_src, void* stream) {
    if (check_batch(map, keys, n)) return 1;
    if (n > map->capacity) ASH_FAIL("more pairs than capacity");
    if (n > 0 && indices == nullptr) ASH_FAIL("null indices pointer");
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (is_capturing(s)) ASH_FAIL("ash_map_load cannot be captured into a graph");
    if (clear_table(map, s, false, static_cast<int32_t>(n))) return 1;
    map->heap_dirty = true;   // the heap is the caller's from here on
    map->counters_known = false;
    map->late_pending = false;
    map->maybe_tombstones = false;
    map->unread_inserts = 0;
    if (heap_src != nullptr && heap_src != map->d.heap) {
        ASH_HIP(hipMemcpyAsync(map->d.heap, heap_src,
                               static_cast<size_t>(map->capacity) * 4,
                               hipMemcpyDeviceToDevice, s));
    }
    // later inserts take their indices from this heap unchecked: entries that
    // address no row are counted with the pairs the load refuses
    check_heap_kernel<<<looping_grid(map->capacity), kBlock, 0, s>>>(map->d.heap, map->capacity,
                                                                   map->d.ctr);
    ASH_LAUNCH_CHECK();
    if (n == 0) return 0;
    ValueArgs va = {};
    return launch_insert<kInsertLoad>(map, keys, n, va, nullptr, indices, s);
}

}  // extern "C"
