// Bulk insert (and erase) of libash_hip.so: builds the table in LDS instead of
// claiming slots with one global compare-and-swap per key.
//
// The per-key kernel (ash_map.hip) is bound by the rate at which the device
// executes atomics on random lines.  When a batch is of the order of the table
// itself it is cheaper to stream: the batch is split by bucket range in two
// coalesced passes (coarse bins, then partitions of 512 buckets inside each
// bin), and one workgroup per partition then owns 64 KB of the table
// exclusively: it loads that range into LDS (or starts from an empty one),
// inserts its records with LDS compare-and-swap and writes the range back with
// full-line stores.
//
// Two ways of handing out indices, both with the reference's heap protocol
// (ash/src/hashmap_gpu.cuh:211-232: a new key takes heap[counter++]):
//
//  * keys only: records are bare 64-bit key codes; the build pass ranks the
//    winners of a partition and takes their indices with one update of the
//    heap counter.
//
//  * keys with value rows ("provisional" indices): moving the rows through the
//    two split passes would triple their traffic, so they never travel.  Row i
//    of the batch is promised heap position base + i (base = the counter on
//    entry) and records are (code, i) pairs of 12 bytes.  If every key turns
//    out to be new the promise holds and the value rows are copied in input
//    order, source and destination both contiguous.  Keys that lose (already
//    stored, repeated inside the batch, or handed to the per-key kernel) leave
//    holes among the promised positions; with U winners the positions
//    base .. base + U - 1 must be the ones in use, so every winner at or beyond
//    base + U ("high" winner) is moved into a hole below it -- there are
//    exactly as many of one as of the other.  A flag byte per row tells losers
//    from winners; the value copy skips losers, and when rows lost two small
//    kernels list the holes and re-point the high winners' slots and copy
//    their rows.  Rows of keys that are not inserted are never written.
//
// Bins and partitions have a fixed capacity (expected count + ten standard
// deviations); what does not fit -- duplicates piled on one key, unpackable
// keys, rows beyond the capacity of the heap -- is put on a spill list and
// handled afterwards by the per-key kernel, so the result is the same map for
// any input.  (A probe sequence stays inside its partition by the table's own
// rule, ash_table.h: next_bucket.)
#include "ash_table.h"

#include "../../include/ash_hip.h"

#include <cmath>

namespace ash {
namespace {

// A build workgroup owns one probe range of the table: kPartBuckets buckets
// (ash_dev.h), the range a probe sequence never leaves.
// Chunk geometry measured on 16 M keys (ms per insert): 1024x4 1.03,
// 1024x2 1.06, 512x4 1.13, 512x8 1.17, 256x8 1.29.
constexpr int kSplitThreads = 1024;
constexpr int kSplitKeys = 4;                   // records per thread
constexpr int kSplitChunk = kSplitThreads * kSplitKeys;
constexpr int kMaxBins = 256;
constexpr int kBuildThreads = 512;
constexpr int kBuildRecs = 4;                   // records per thread and round
constexpr int kCopyThreads = 256;
constexpr int64_t kMinKeys = 1 << 12;

// Header words at the start of the workspace.
enum { kHdrSpillKeys = 0, kHdrSpillA = 1, kHdrWasEmpty = 3,
       kHdrBase = 4,      // heap counter on entry
       kHdrLosers = 5,    // rows that did not win a slot in the build pass
       kHdrHoles = 6,     // listed holes
       kHdrTaken = 7,     // holes handed to high winners
       kHdrTicket = 8,    // workgroups of pass 1 that are done
       kHdrWords = 64 };

struct BulkPlan {
    int64_t n;
    uint32_t parts;        // partitions of kPartBuckets buckets
    uint32_t bins;         // coarse bins of (1 << fine_shift) partitions
    uint32_t fine_shift;
    // A coarse bin's buffer consists of 1 << lane_shift lanes with a cursor
    // each; workgroup w of pass 1 appends to lane w mod lanes.  Every chunk of
    // pass 1 reserves a run in every bin, and updates of one address serialise
    // (about 7 ns each): with one cursor per bin the 3906 chunks of 16 M keys
    // queued for 27 us at each, a quarter of the pass.
    uint32_t lane_shift;
    uint32_t cap_bin;      // records per lane of a coarse bin
    uint32_t cap_part;     // records per partition
    uint32_t chunks;       // split chunks per lane of a coarse bin
    int32_t* hdr;
    int32_t* cursor_bin;   // bins << lane_shift
    int32_t* cursor_part;  // bins << fine_shift
    uint64_t* codes_a;     // (bins << lane_shift) * cap_bin
    uint64_t* codes_b;     // parts * cap_part
    // keys only
    int32_t* spill_keys;   // n input row numbers (also the one list of the provisional scheme)
    int32_t* spill_a;      // n positions in the coarse plane
    // provisional scheme
    int32_t* rows_a;       // bins * cap_bin input row numbers
    int32_t* rows_b;       // parts * cap_part
    uint8_t* flags;        // n: 1 = row i did not win a slot
    int32_t* holes;        // n / 2 + 64 row numbers
};

inline int64_t align256(int64_t x) { return (x + 255) & ~int64_t{255}; }

// Fills `pl` for `n` keys; returns the workspace size, or 0 when the bulk path
// does not apply.  With ws == nullptr only sizes are computed.
int64_t make_plan(const ash_map* map, int64_t n, int n_values,
                  const int64_t* row_bytes, char* ws, BulkPlan& pl) {
    if (n < kMinKeys || n_values < 0 || n_values > kMaxFusedValues) return 0;
    for (int v = 0; v < n_values; ++v) {
        if (row_bytes[v] <= 0 || row_bytes[v] % 4 != 0 ||
            row_bytes[v] > kMaxFusedRowDwords * 4) {
            return 0;
        }
    }
    const int64_t nb = map->d.nb;
    const int64_t parts = (nb + kPartBuckets - 1) >> kPartShift;
    uint32_t fine_shift = 6;
    while (fine_shift < 8 && ((parts + (1ll << fine_shift) - 1) >> fine_shift) > kMaxBins) {
        ++fine_shift;
    }
    const int64_t bins = (parts + (1ll << fine_shift) - 1) >> fine_shift;
    if (bins > kMaxBins) return 0;
    const double per_bucket = static_cast<double>(n) / static_cast<double>(nb);
    double mean_bin = per_bucket * kPartBuckets * static_cast<double>(1ll << fine_shift);
    const double mean_part = per_bucket * kPartBuckets;
    // lanes per bin: as many (up to eight) as leave a lane two chunks of pass 2
    uint32_t lane_shift = 0;
    while (lane_shift < 3 && mean_bin >= 4.0 * kSplitChunk) {
        ++lane_shift;
        mean_bin *= 0.5;
    }
    int64_t cap_bin = static_cast<int64_t>(mean_bin + 10.0 * std::sqrt(mean_bin)) + 256;
    int64_t cap_part = static_cast<int64_t>(mean_part + 10.0 * std::sqrt(mean_part)) + 64;
    if (cap_bin > n) cap_bin = n;
    if (cap_part > n) cap_part = n;
    cap_bin = (cap_bin + 15) & ~int64_t{15};
    cap_part = (cap_part + 15) & ~int64_t{15};
    const int64_t na = (bins << lane_shift) * cap_bin;
    const int64_t nbp = parts * cap_part;
    if (na >= (int64_t{1} << 31) || nbp >= (int64_t{1} << 31)) return 0;

    pl.n = n;
    pl.parts = static_cast<uint32_t>(parts);
    pl.bins = static_cast<uint32_t>(bins);
    pl.fine_shift = fine_shift;
    pl.lane_shift = lane_shift;
    pl.cap_bin = static_cast<uint32_t>(cap_bin);
    pl.cap_part = static_cast<uint32_t>(cap_part);
    pl.chunks = static_cast<uint32_t>((cap_bin + kSplitChunk - 1) / kSplitChunk);

    int64_t off = 0;
    auto take = [&](int64_t bytes) {
        char* p = ws ? ws + off : nullptr;
        off += align256(bytes);
        return p;
    };
    pl.hdr = reinterpret_cast<int32_t*>(take(kHdrWords * 4));
    pl.cursor_bin = reinterpret_cast<int32_t*>(take((bins << lane_shift) * 4));
    pl.cursor_part = reinterpret_cast<int32_t*>(take((bins << fine_shift) * 4));
    pl.codes_a = reinterpret_cast<uint64_t*>(take(na * 8));
    pl.codes_b = reinterpret_cast<uint64_t*>(take(nbp * 8));
    pl.spill_keys = reinterpret_cast<int32_t*>(take(n * 4));
    pl.spill_a = nullptr;
    pl.rows_a = pl.rows_b = pl.holes = nullptr;
    pl.flags = nullptr;
    if (n_values == 0) {
        pl.spill_a = reinterpret_cast<int32_t*>(take(n * 4));
    } else {
        pl.rows_a = reinterpret_cast<int32_t*>(take(na * 4));
        pl.rows_b = reinterpret_cast<int32_t*>(take(nbp * 4));
        pl.flags = reinterpret_cast<uint8_t*>(take(n));
        pl.holes = reinterpret_cast<int32_t*>(take((n / 2 + 64) * 4));
    }
    return off;
}

// ------------------------------------------------------------- kernels
__global__ void bulk_init_kernel(MapDev m, BulkPlan pl, int ncursors) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    // cursor_bin and cursor_part are zeroed separately: they are not adjacent
    if (t < static_cast<int>(pl.bins << pl.lane_shift)) pl.cursor_bin[t] = 0;
    if (t < ncursors) pl.cursor_part[t] = 0;
    if (t < kHdrWords) {
        int32_t v = 0;
        if (t == kHdrWasEmpty) v = (m.ctr[kCtrSize] == 0 && m.ctr[kCtrTombs] == 0) ? 1 : 0;
        if (t == kHdrBase) v = m.ctr[kCtrSize];
        pl.hdr[t] = v;
    }
}

// Rows of the batch that can be promised a heap position.
__device__ __forceinline__ int64_t rows_that_fit(const MapDev& m, const BulkPlan& pl) {
    const int64_t room = static_cast<int64_t>(m.capacity) - pl.hdr[kHdrBase];
    return room < 0 ? 0 : (room < pl.n ? room : pl.n);
}

// LDS of the two split passes.  Every record of the workgroup's chunk gets a
// bin and its arrival rank inside that bin (LDS counter); reserve_runs turns
// the counts into start[b] (first sorted position of bin b inside the chunk)
// and base[b] (position of the chunk's run inside the bin's global buffer,
// reserved with one atomic per bin).  Each thread then drops its records at
// their sorted positions in `stage`, and the workgroup writes the stage out
// front to back, so that global reads and writes both have consecutive lanes
// on consecutive records.
struct SplitShared {
    int cnt[kMaxBins];
    int start[kMaxBins];
    int base[kMaxBins];
    int wave_total[kMaxBins / 64];
    int losers;
    int nspill;        // rows of this chunk that pass 1 leaves to the per-key kernel
    int spill_first;   // their place in the spill list
    // sorted position -> input row (provisional scheme) or record of the chunk
    int32_t aux[kSplitChunk];
    uint8_t bin_of[kSplitChunk];   // sorted position -> bin
    uint64_t stage[kSplitChunk];   // sorted position -> code
};

// `shift`, `lane`: the cursor of bin b is cursors[(b << shift) + lane].
__device__ __forceinline__ int reserve_runs(SplitShared& sh, int32_t* cursors,
                                            int nbins, int shift = 0, int lane_of_bin = 0) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    int v = 0, incl = 0;
    if (tid < kMaxBins) {
        v = sh.cnt[tid];
        incl = v;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(incl, d);
            if (lane >= d) incl += up;
        }
        if (lane == 63) sh.wave_total[tid >> 6] = incl;
    }
    __syncthreads();
    if (tid < kMaxBins) {
        int off = 0;
        for (int w = 0; w < (tid >> 6); ++w) off += sh.wave_total[w];
        sh.start[tid] = off + incl - v;
        sh.base[tid] = (v && tid < nbins) ? atomicAdd(cursors + (tid << shift) + lane_of_bin, v) : 0;
    }
    __syncthreads();
    int total = 0;
#pragma unroll
    for (int w = 0; w < kMaxBins / 64; ++w) total += sh.wave_total[w];
    return total;
}

// Moves the ranked records of a chunk to their runs.  code/aux/bin/rank
// describe the calling thread's kSplitKeys records (bin < 0 = not taking
// part); aux is what travels with the code: the input row in the provisional
// scheme (written to aux_dst), the record's number inside the chunk otherwise
// (only used to name a record that does not fit).  Destination of a record
// with bin b and position pos inside the bin: dst_first(b) + pos, valid while
// pos < cap; the others are reported through `spill` with their aux value.
template <bool PROV, typename DstFirst, typename Spill>
__device__ __forceinline__ void move_chunk(
        SplitShared& sh, int total, const uint64_t (&code)[kSplitKeys],
        const int32_t (&aux)[kSplitKeys], const int (&bin)[kSplitKeys],
        const int (&rank)[kSplitKeys], uint64_t* __restrict__ codes_dst,
        int32_t* __restrict__ aux_dst, uint32_t cap, DstFirst dst_first, Spill spill) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int k = 0; k < kSplitKeys; ++k) {
        if (bin[k] >= 0) {
            const int sp = sh.start[bin[k]] + rank[k];
            sh.aux[sp] = aux[k];
            sh.bin_of[sp] = static_cast<uint8_t>(bin[k]);
            sh.stage[sp] = code[k];
        }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kSplitKeys; ++j) {
        const int s = j * kSplitThreads + tid;
        if (s < total) {
            const int b = sh.bin_of[s];
            const uint32_t pos =
                    static_cast<uint32_t>(sh.base[b] + (s - sh.start[b]));
            if (pos < cap) {
                const int64_t d = dst_first(b) + pos;
                codes_dst[d] = sh.stage[s];
                if constexpr (PROV) aux_dst[d] = sh.aux[s];
            } else {
                spill(sh.aux[s]);
            }
        }
    }
}

// A row of the provisional scheme that will not be placed by the build pass:
// flagged, counted, and (unless it is a plain duplicate) left to the per-key
// kernel.
__device__ __forceinline__ void give_up_row(const BulkPlan& pl, int32_t row, int* losers,
                                            bool to_per_key_kernel) {
    pl.flags[row] = 1;
    atomicAdd(losers, 1);
    if (to_per_key_kernel) pl.spill_keys[atomicAdd(pl.hdr + kHdrSpillKeys, 1)] = row;
}

// Pass 1: input rows -> coarse bins, 4096 keys per workgroup.
// `identity` (provisional scheme): the heap is 0, 1, 2, ..., so row i's promised
// index is base + i and the key log can be written here, in input order; with a
// heap in another order the build pass writes it.
template <int DIM, bool PROV>
__global__ __launch_bounds__(kSplitThreads) void split_keys_kernel(
        MapDev m, BulkPlan pl, const int32_t* __restrict__ keys, int identity,
        int32_t* __restrict__ early) {
    __shared__ SplitShared sh;
    const int tid = threadIdx.x;
    if (tid < kMaxBins) sh.cnt[tid] = 0;
    if (tid == 0) {
        sh.losers = 0;
        sh.nspill = 0;
    }
    __syncthreads();
    const int64_t base = static_cast<int64_t>(blockIdx.x) * kSplitChunk;
    const int bin_shift = kPartShift + static_cast<int>(pl.fine_shift);
    const int64_t fit = PROV ? rows_that_fit(m, pl) : pl.n;
    const int64_t heap_base = PROV ? pl.hdr[kHdrBase] : 0;
    uint64_t code[kSplitKeys];
    int32_t aux[kSplitKeys];
    int bin[kSplitKeys];
    int rank[kSplitKeys];
    int spill_rank[kSplitKeys];
#pragma unroll
    for (int k = 0; k < kSplitKeys; ++k) {
        const int64_t i = base + k * kSplitThreads + tid;
        const bool active = i < pl.n;
        int32_t key[DIM];
        load_key<DIM>(keys, i, active, key);
        const bool fits = pack_key<DIM>(key, code[k]);
        bin[k] = -1;
        rank[k] = 0;
        spill_rank[k] = -1;
        aux[k] = PROV ? static_cast<int32_t>(i) : k * kSplitThreads + tid;
        if (active && fits && i < fit) {
            bin[k] = static_cast<int>(bucket_of(code[k], m.nb) >> bin_shift);
            rank[k] = atomicAdd(&sh.cnt[bin[k]], 1);
            if constexpr (PROV) {
                pl.flags[i] = 0;
                if (identity) __builtin_nontemporal_store(code[k], m.klog + heap_base + i);
            }
        } else if (active) {
            // unpackable, or beyond what the heap can still give: left to the
            // per-key kernel (listed below, one update of the list's counter
            // per workgroup: a batch far beyond the capacity lands here)
            spill_rank[k] = atomicAdd(&sh.nspill, 1);
            if constexpr (PROV) pl.flags[i] = 1;
        }
    }
    __syncthreads();
    if (tid == 0 && sh.nspill) {
        sh.spill_first = atomicAdd(pl.hdr + kHdrSpillKeys, sh.nspill);
        if constexpr (PROV) sh.losers = sh.nspill;
    }
    const int my_lane = static_cast<int>(blockIdx.x & ((1u << pl.lane_shift) - 1u));
    const int total = reserve_runs(sh, pl.cursor_bin, static_cast<int>(pl.bins),
                                   static_cast<int>(pl.lane_shift), my_lane);
#pragma unroll
    for (int k = 0; k < kSplitKeys; ++k) {
        if (spill_rank[k] >= 0) {
            pl.spill_keys[sh.spill_first + spill_rank[k]] =
                    static_cast<int32_t>(base + k * kSplitThreads + tid);
        }
    }
    move_chunk<PROV>(
            sh, total, code, aux, bin, rank, pl.codes_a, pl.rows_a, pl.cap_bin,
            [&](int b) {
                return static_cast<int64_t>((static_cast<uint32_t>(b) << pl.lane_shift) + my_lane) *
                       pl.cap_bin;
            },
            [&](int32_t a) {
                if constexpr (PROV) {
                    give_up_row(pl, a, &sh.losers, true);
                } else {
                    pl.spill_keys[atomicAdd(pl.hdr + kHdrSpillKeys, 1)] =
                            static_cast<int32_t>(base + a);
                }
            });
    if constexpr (PROV) {
        __syncthreads();
        if (tid == 0 && sh.losers) atomicAdd(pl.hdr + kHdrLosers, sh.losers);
    }
    if (early != nullptr) {
        // `early`: page-locked host memory.  The workgroup that finishes last
        // leaves there how many rows this pass has handed to the per-key
        // kernel, for a host that waits for nothing else of the call.  (Every
        // update of that count has returned its value to the thread that made
        // it before the barrier; no fence: one per wavefront would write the
        // L2 back each time, which multiplied the duration of this pass.)
        __syncthreads();
        if (tid == 0 &&
            atomicAdd(pl.hdr + kHdrTicket, 1) == static_cast<int32_t>(gridDim.x) - 1) {
            __hip_atomic_store(early, atomicAdd(pl.hdr + kHdrSpillKeys, 0), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_SYSTEM);
            __threadfence_system();
        }
    }
}

// Pass 2: coarse bin -> partitions.  Workgroup (bin, lane, chunk) takes 4096
// records of its lane of the bin.
template <bool PROV>
__global__ __launch_bounds__(kSplitThreads) void split_records_kernel(MapDev m, BulkPlan pl) {
    __shared__ SplitShared sh;
    const int tid = threadIdx.x;
    const uint32_t lane_of_bin = blockIdx.x / pl.chunks;   // (bin << lane_shift) + lane
    const uint32_t chunk = blockIdx.x % pl.chunks;
    const uint32_t c = lane_of_bin >> pl.lane_shift;
    int cnt = pl.cursor_bin[lane_of_bin];
    if (cnt > static_cast<int>(pl.cap_bin)) cnt = static_cast<int>(pl.cap_bin);
    const int start = static_cast<int>(chunk) * kSplitChunk;
    if (start >= cnt) return;
    if (tid < kMaxBins) sh.cnt[tid] = 0;
    if (tid == 0) sh.losers = 0;
    __syncthreads();
    const int64_t abase = static_cast<int64_t>(lane_of_bin) * pl.cap_bin + start;
    const uint32_t fmask = (1u << pl.fine_shift) - 1u;
    uint64_t code[kSplitKeys];
    int32_t aux[kSplitKeys];
    int bin[kSplitKeys];
    int rank[kSplitKeys];
#pragma unroll
    for (int k = 0; k < kSplitKeys; ++k) {
        const int j = k * kSplitThreads + tid;
        bin[k] = -1;
        rank[k] = 0;
        code[k] = 0;
        aux[k] = j;
        if (start + j < cnt) {
            // (records are read once: loads marked as not to be kept in the
            // caches, here and in the range passes; 3 % of an insert)
            code[k] = __builtin_nontemporal_load(pl.codes_a + abase + j);
            if constexpr (PROV) aux[k] = __builtin_nontemporal_load(pl.rows_a + abase + j);
            bin[k] = static_cast<int>((bucket_of(code[k], m.nb) >> kPartShift) & fmask);
            rank[k] = atomicAdd(&sh.cnt[bin[k]], 1);
        }
    }
    __syncthreads();
    const int total = reserve_runs(
            sh, pl.cursor_part + (static_cast<size_t>(c) << pl.fine_shift),
            static_cast<int>(fmask) + 1);
    move_chunk<PROV>(
            sh, total, code, aux, bin, rank, pl.codes_b, pl.rows_b, pl.cap_part,
            [&](int b) {
                return static_cast<int64_t>((c << pl.fine_shift) +
                                            static_cast<uint32_t>(b)) *
                       pl.cap_part;
            },
            [&](int32_t a) {
                if constexpr (PROV) {
                    give_up_row(pl, a, &sh.losers, true);
                } else {
                    pl.spill_a[atomicAdd(pl.hdr + kHdrSpillA, 1)] =
                            static_cast<int32_t>(abase + a);
                }
            });
    if constexpr (PROV) {
        __syncthreads();
        if (tid == 0 && sh.losers) atomicAdd(pl.hdr + kHdrLosers, sh.losers);
    }
}

// Where the q-th 16 bytes of local bucket lb sit in the LDS copy of the table
// range.  A bucket is 128 bytes = 32 banks wide, so without the rotation every
// lane that reads "16 bytes number q of its bucket" would hit the same four
// banks; rotating by the bucket number spreads them over all of them.
__device__ __forceinline__ int staged(int lb, int q) {
    return lb * kGroup + ((q + lb) & (kGroup - 1));
}

enum { kPlaced = 0, kKnown = 1, kFull = 2 };

// Inserts `code` into the LDS copy of the partition, starting at local bucket
// lb and going round inside the partition (next_bucket's rule).  kPlaced: the
// calling thread owns slot `where` (local bucket * 16 + slot) now; kKnown: the
// code was there already (or another thread of this round placed it); kFull:
// every bucket of the partition has been visited.
__device__ __forceinline__ int place_code(uint4* tab, uint64_t code, int lb, int nbk,
                                          int& where) {
    unsigned long long* tab64 = reinterpret_cast<unsigned long long*>(tab);
    for (int visited = 0; visited < nbk; ++visited) {
        uint64_t c[kSlots];
#pragma unroll
        for (int q = 0; q < kSlots / 2; ++q) {
            const uint4 w = tab[staged(lb, q)];
            c[2 * q] = static_cast<uint64_t>(w.x) | (static_cast<uint64_t>(w.y) << 32);
            c[2 * q + 1] = static_cast<uint64_t>(w.z) | (static_cast<uint64_t>(w.w) << 32);
        }
        bool known = false;
        uint32_t em = 0;
#pragma unroll
        for (int s = 0; s < kSlots; ++s) {
            known |= c[s] == code;
            em |= (c[s] == kEmpty ? 1u : 0u) << s;
        }
        if (known) return kKnown;
        while (em) {
            const int s = __builtin_ctz(em);
            const unsigned long long old =
                    atomicCAS(tab64 + staged(lb, s >> 1) * 2 + (s & 1), kEmpty, code);
            if (old == kEmpty) {
                where = lb * kBucketQwords + s;
                return kPlaced;
            }
            if (old == code) return kKnown;
            em &= em - 1;
        }
        if (++lb == nbk) lb = 0;
    }
    return kFull;
}

// Among the first n slots of local bucket lb (n <= kSlots, all of them
// written), empties every slot that holds the code of a lower slot; `dropped`
// is told the slot before it is emptied.  Every lane of the wavefront calls
// this (n = 0: nothing to look at).
template <typename Dropped>
__device__ __forceinline__ void drop_repeats(uint4* tab, int lb, int n, Dropped dropped) {
    uint64_t c[kSlots];
#pragma unroll
    for (int q = 0; q < kSlots / 2; ++q) {
        const uint4 w = n > 2 * q ? tab[staged(lb, q)] : make_uint4(0u, 0u, 0u, 0u);
        c[2 * q] = static_cast<uint64_t>(w.x) | (static_cast<uint64_t>(w.y) << 32);
        c[2 * q + 1] = static_cast<uint64_t>(w.z) | (static_cast<uint64_t>(w.w) << 32);
    }
    // low words first: two slots hold the same code only if they agree there,
    // which is rare enough to let whole wavefronts skip the full comparison
    // (slots from n on get low words of their own)
    uint32_t lo[kSlots];
#pragma unroll
    for (int j = 0; j < kSlots; ++j) lo[j] = j < n ? static_cast<uint32_t>(c[j]) : 0x80000000u + j;
    bool maybe = false;
#pragma unroll
    for (int j = 1; j < kSlots; ++j) {
#pragma unroll
        for (int i = 0; i < j; ++i) maybe = maybe || lo[i] == lo[j];
    }
    if (!__ballot(maybe)) return;
    uint32_t repeat = 0;
#pragma unroll
    for (int j = 1; j < kSlots; ++j) {
#pragma unroll
        for (int i = 0; i < j; ++i) {
            // (a slot emptied by an earlier look is not a copy of another such slot)
            if (lo[i] == lo[j] && c[i] == c[j] && j < n && c[j] != kEmpty) repeat |= 1u << j;
        }
    }
    unsigned long long* tab64 = reinterpret_cast<unsigned long long*>(tab);
    while (repeat) {
        const int j = __builtin_ctz(repeat);
        dropped(j);
        tab64[staged(lb, j >> 1) * 2 + (j & 1)] = kEmpty;
        repeat &= repeat - 1;
    }
}

// Pass 3: one workgroup per partition builds its 512 buckets in LDS.
// `stale`: the bucket array holds leftovers of a table that has been cleared
// since (the clear left the fill to its successor): every partition is then
// written, those without records as empty ones.  `identity`: the heap is
// 0, 1, 2, ... (nothing has written to it since it was last reset), so
// position p holds index p and need not be read.
//
// Into a range that starts empty (the map was empty on entry) records are
// placed by counting: a record draws a number in its bucket (one LDS atomic)
// and, while that number is below the bucket's ten slots, simply writes its
// code there -- no read of the bucket, no compare-and-swap.  Copies of one key
// draw different numbers in the same bucket: after a barrier one thread per
// bucket compares the codes written so far and empties every slot that repeats
// a lower one (a wavefront reads 64 whole buckets per instruction; a look by
// every record at the slots below its own costs as many LDS instructions as
// the probing path).  When a record's index is known as it draws (provisional
// scheme, heap in its initial order) it is stored with the code and tells the
// comparing thread which row lost; otherwise, after another barrier, a record
// that no longer finds its code in its slot has lost.  Records whose number is ten or more (a
// crowded bucket, or many copies of few keys) wait until every record of the
// partition has drawn and are then placed by the probing path, which first
// looks into the home bucket like any probe.  That path alone serves a range
// that holds entries already.
enum { kRecIdle = 0, kRecPlaced = 1, kRecLost = 2 };
constexpr int kWaitList = 128;

template <bool PROV>
__global__ __launch_bounds__(kBuildThreads) void build_kernel(
        MapDev m, BulkPlan pl, int stale, int identity) {
    // Records per thread and round.  With rows the partitions of a batch of the
    // order of the table take one round of five (16 M keys into 24 M: 2048 +- 45
    // records per partition; with four, half of the partitions went through
    // every phase twice, 162 against 139 us); keys only, a fifth record costs
    // more in the ranking of the winners than the second round (262 against
    // 185 us).
    constexpr int kRecs = PROV ? 5 : kBuildRecs;
    constexpr int kRound = kBuildThreads * kRecs;
    constexpr int kCountedRounds = 32 / kRecs;   // one bit per record of a thread
    constexpr int kRecSlots = kRecs + 1;
    __shared__ uint4 tab[kPartBuckets * kGroup];
    // winners per (record slot k, wavefront), then their exclusive prefix
    __shared__ int s_wcnt[kRecSlots * (kBuildThreads / 64)];
    __shared__ int s_base;
    __shared__ int s_losers;
    __shared__ int s_drawn[kPartBuckets];   // numbers drawn per bucket (range that starts empty)
    __shared__ int s_seen[kPartBuckets];    // of which drop_repeats has compared this many
    // records that wait for the probing path: the first kWaitList of them here,
    // the others are read again from the partition's records
    __shared__ uint64_t s_wait_code[kWaitList];
    __shared__ int32_t s_wait_row[kWaitList];
    __shared__ int s_nwait;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const uint32_t p = blockIdx.x;
    int cnt = pl.cursor_part[p];
    if (cnt > static_cast<int>(pl.cap_part)) cnt = static_cast<int>(pl.cap_part);
    const uint32_t b0 = p << kPartShift;
    if (b0 >= m.nb) return;
    const int nbk = static_cast<int>(m.nb - b0 < static_cast<uint32_t>(kPartBuckets)
                                             ? m.nb - b0
                                             : static_cast<uint32_t>(kPartBuckets));
    uint4* __restrict__ gl =
            reinterpret_cast<uint4*>(m.buckets) + static_cast<size_t>(b0) * kGroup;
    if (cnt == 0) {
        if (stale) {
            for (int t = tid; t < nbk * kGroup; t += kBuildThreads) {
                gl[t] = make_uint4(~0u, ~0u, ~0u, ~0u);
            }
        }
        return;
    }
    const bool was_empty = pl.hdr[kHdrWasEmpty] != 0;
    const bool counted = was_empty && cnt <= kCountedRounds * kRound;
    const int32_t heap_base = pl.hdr[kHdrBase];
    const int64_t bbase = static_cast<int64_t>(p) * pl.cap_part;
    if (tid == 0) {
        s_losers = 0;
        s_nwait = 0;
    }
    // (slot kRecs: a record taken from the waiting list, last round only)
    uint64_t codes[kRecSlots] = {};
    int32_t rows[kRecSlots] = {};
    // records rb + k * kBuildThreads + tid, k < kRecs; with `only`, just
    // those whose bit is set
    auto load_round = [&](int rb, uint32_t only) {
#pragma unroll
        for (int k = 0; k < kRecs; ++k) {
            const int r = rb + k * kBuildThreads + tid;
            const bool take = r < cnt && ((only >> k) & 1u);
            codes[k] = take ? __builtin_nontemporal_load(pl.codes_b + bbase + r) : 0ull;
            if constexpr (PROV) rows[k] = take ? __builtin_nontemporal_load(pl.rows_b + bbase + r) : 0;
        }
    };
    // The first round's records are requested before the table range is
    // staged, so that both latencies overlap.
    load_round(0, ~0u);
    for (int t = tid; t < nbk * kGroup; t += kBuildThreads) {
        tab[staged(t >> 3, t & 7)] =
                was_empty ? make_uint4(~0u, ~0u, ~0u, ~0u) : gl[t];
    }
    for (int t = tid; t < static_cast<int>(kPartBuckets); t += kBuildThreads) {
        s_drawn[t] = 0;
        s_seen[t] = 0;
    }
    __syncthreads();

    unsigned long long* tab64 = reinterpret_cast<unsigned long long*>(tab);
    int32_t* tab32 = reinterpret_cast<int32_t*>(tab);
    auto store_index = [&](int where, int32_t idx) {
        const int wlb = where >> 4;
        const int ws = where & 15;
        tab32[staged(wlb, (kValDword0 + ws) >> 2) * 4 + (ws & 3)] = idx;
    };
    auto code_at = [&](int where) -> unsigned long long& {
        return tab64[staged(where >> 4, (where & 15) >> 1) * 2 + (where & 1)];
    };

    // Indices for the records of a round that hold a slot (state kRecPlaced,
    // slot in wslot); rows of the provisional scheme that did not get one
    // (kRecLost) are given up.  Every thread calls this the same number of times.
    auto settle_round = [&](const int (&state)[kRecSlots], const int (&wslot)[kRecSlots]) {
        if constexpr (PROV) {
#pragma unroll
            for (int k = 0; k < kRecSlots; ++k) {
                if (state[k] == kRecPlaced) {
                    // the promised position; re-pointed later if it turns out
                    // to lie beyond the last position in use
                    const int32_t pos = heap_base + rows[k];
                    if (identity) {
                        store_index(wslot[k], pos);   // the log was written by pass 1
                    } else {
                        const int32_t idx = m.heap[pos];
                        store_index(wslot[k], idx);
                        m.klog[idx] = codes[k];
                    }
                } else if (state[k] == kRecLost) {
                    give_up_row(pl, rows[k], &s_losers, false);
                }
            }
        } else {
            // Winners are ranked in record order, so that consecutive lanes
            // take consecutive heap entries.
            int wrank[kRecSlots];
#pragma unroll
            for (int k = 0; k < kRecSlots; ++k) {
                const uint64_t wm = __ballot(state[k] == kRecPlaced);
                wrank[k] = __popcll(wm & ((1ull << lane) - 1ull));
                if (lane == 0) s_wcnt[k * (kBuildThreads / 64) + wave] = __popcll(wm);
            }
            __syncthreads();
            if (tid == 0) {
                int tot = 0;
                for (int q = 0; q < kRecSlots * (kBuildThreads / 64); ++q) {
                    const int c = s_wcnt[q];
                    s_wcnt[q] = tot;
                    tot += c;
                }
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
#pragma unroll
            for (int k = 0; k < kRecSlots; ++k) {
                if (state[k] != kRecPlaced) continue;
                const int top = s_base + s_wcnt[k * (kBuildThreads / 64) + wave] + wrank[k];
                if (top < m.capacity) {
                    const int32_t idx = identity ? top : m.heap[top];
                    store_index(wslot[k], idx);
                    m.klog[idx] = codes[k];
                } else {
                    // Heap exhausted: give the slot up again.
                    code_at(wslot[k]) = kTomb;
                    atomicAdd(m.ctr + kCtrTombs, 1);
                }
            }
        }
        __syncthreads();
    };
    // The probing path for the records of a round whose bit is set in `which`.
    auto probe_round = [&](uint32_t which, int (&state)[kRecSlots], int (&wslot)[kRecSlots]) {
#pragma unroll
        for (int k = 0; k < kRecSlots; ++k) {
            state[k] = kRecIdle;
            wslot[k] = -1;
            if (!((which >> k) & 1u)) continue;
            const int lb = static_cast<int>(bucket_of(codes[k], m.nb) - b0);
            const int how = place_code(tab, codes[k], lb, nbk, wslot[k]);
            if (how == kFull) atomicAdd(m.ctr + kCtrDropped, 1);   // refused
            state[k] = how == kPlaced ? kRecPlaced : kRecLost;
        }
    };

    // the index of a record is known when it draws its number
    const bool direct = PROV && identity != 0;
    uint32_t waiting = 0;   // bit round * kRecs + k: that record drew a number beyond the slots
    int round = 0;
    for (int rb = 0; rb < cnt; rb += kRound, ++round) {
        int wslot[kRecSlots];
        int state[kRecSlots];
        if (rb > 0) load_round(rb, ~0u);
        state[kRecs] = kRecIdle;
        wslot[kRecs] = -1;
        uint32_t live = 0;
#pragma unroll
        for (int k = 0; k < kRecs; ++k) {
            if (rb + k * kBuildThreads + tid < cnt) live |= 1u << k;
        }
        if (!counted) {
            probe_round(live, state, wslot);
        } else {
#pragma unroll
            for (int k = 0; k < kRecs; ++k) {
                state[k] = kRecIdle;
                wslot[k] = -1;
                if (!((live >> k) & 1u)) continue;
                const int lb = static_cast<int>(bucket_of(codes[k], m.nb) - b0);
                const int number = atomicAdd(&s_drawn[lb], 1);
                if (number < kSlots) {
                    wslot[k] = lb * kBucketQwords + number;
                    code_at(wslot[k]) = codes[k];
                    state[k] = kRecPlaced;
                    if (direct) {
                        store_index(wslot[k], heap_base + rows[k]);
                        state[k] = kRecIdle;   // nothing left to do for it
                    }
                } else {
                    const int at = atomicAdd(&s_nwait, 1);
                    if (at < kWaitList) {
                        s_wait_code[at] = codes[k];
                        s_wait_row[at] = rows[k];
                    } else {
                        waiting |= 1u << (round * kRecs + k);
                    }
                }
            }
            __syncthreads();
            for (int first = 0; first < nbk; first += kBuildThreads) {
                const int lb = first + tid;
                int drawn = 0;
                if (lb < nbk) {
                    drawn = s_drawn[lb] < kSlots ? s_drawn[lb] : kSlots;
                    // (numbers drawn in earlier rounds have been looked at)
                    const bool news = drawn >= 2 && drawn > s_seen[lb];
                    s_seen[lb] = drawn;
                    if (!news) drawn = 0;
                }
                drop_repeats(tab, lb < nbk ? lb : 0, drawn, [&](int j) {
                    if constexpr (PROV) {
                        if (direct) {
                            const int32_t idx = tab32[staged(lb, (kValDword0 + j) >> 2) * 4 + (j & 3)];
                            give_up_row(pl, idx - heap_base, &s_losers, false);
                        }
                    }
                });
            }
            const bool last = rb + kRound >= cnt && s_nwait > 0;
            if (!direct || last) __syncthreads();
            if (!direct) {
#pragma unroll
                for (int k = 0; k < kRecs; ++k) {
                    if (state[k] == kRecPlaced && code_at(wslot[k]) != codes[k]) state[k] = kRecLost;
                }
            }
            if (last) {
                // the last round: every record has drawn, so the listed
                // waiting records take the probing path now and get their
                // indices with this round's
                const int listed = s_nwait < kWaitList ? s_nwait : kWaitList;
                if (tid < listed) {
                    constexpr int x = kRecs;
                    codes[x] = s_wait_code[tid];
                    rows[x] = s_wait_row[tid];
                    const int lb = static_cast<int>(bucket_of(codes[x], m.nb) - b0);
                    const int how = place_code(tab, codes[x], lb, nbk, wslot[x]);
                    if (how == kFull) atomicAdd(m.ctr + kCtrDropped, 1);   // refused
                    state[x] = how == kPlaced ? kRecPlaced : kRecLost;
                }
            }
        }
        settle_round(state, wslot);
    }
    // (s_nwait is final: every round ends with a barrier)
    if (counted && s_nwait > kWaitList) {
        round = 0;
        for (int rb = 0; rb < cnt; rb += kRound, ++round) {
            const uint32_t mine = (waiting >> (round * kRecs)) & ((1u << kRecs) - 1u);
            if (!__syncthreads_or(mine != 0)) continue;
            int wslot[kRecSlots];
            int state[kRecSlots];
            load_round(rb, mine);
            probe_round(mine, state, wslot);
            settle_round(state, wslot);
        }
    }
    // (stores marked as not to be kept in the caches: nothing reads the range,
    // the value rows or the log entries again before a later call does; the
    // insert with values of 16 M keys: 0.588 -> 0.570 ms)
    {
        typedef unsigned int v4u __attribute__((ext_vector_type(4)));
        for (int t = tid; t < nbk * kGroup; t += kBuildThreads) {
            const uint4 x = tab[staged(t >> 3, t & 7)];
            v4u y = {x.x, x.y, x.z, x.w};
            __builtin_nontemporal_store(y, reinterpret_cast<v4u*>(gl) + t);
        }
    }
    if constexpr (PROV) {
        if (tid == 0 && s_losers) atomicAdd(pl.hdr + kHdrLosers, s_losers);
    }
}

// Streaming erase, pass 3: one workgroup per partition takes its range of the
// table into LDS, looks its records up there and frees what it finds: the slot
// goes back to empty while its bucket has an empty slot left (such a bucket has
// never been full, so no key was ever pushed past it) and becomes a tombstone
// otherwise -- the rule of the per-key kernel (erase_one, ash_map.hip).  Freed
// indices return to the heap below the counter, which moves once per
// workgroup and round.  A range none of whose records was found is not
// written back.
__global__ __launch_bounds__(kBuildThreads) void erase_range_kernel(MapDev m, BulkPlan pl) {
    __shared__ uint4 tab[kPartBuckets * kGroup];
    __shared__ int s_wcnt[kBuildRecs * (kBuildThreads / 64)];
    __shared__ int s_base;
    __shared__ int s_tombs;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const uint32_t p = blockIdx.x;
    int cnt = pl.cursor_part[p];
    if (cnt > static_cast<int>(pl.cap_part)) cnt = static_cast<int>(pl.cap_part);
    const uint32_t b0 = p << kPartShift;
    if (b0 >= m.nb || cnt == 0) return;
    const int nbk = static_cast<int>(m.nb - b0 < static_cast<uint32_t>(kPartBuckets)
                                             ? m.nb - b0
                                             : static_cast<uint32_t>(kPartBuckets));
    uint4* __restrict__ gl =
            reinterpret_cast<uint4*>(m.buckets) + static_cast<size_t>(b0) * kGroup;
    const int64_t bbase = static_cast<int64_t>(p) * pl.cap_part;
    uint64_t codes[kBuildRecs];
#pragma unroll
    for (int k = 0; k < kBuildRecs; ++k) {
        const int r = k * kBuildThreads + tid;
        codes[k] = r < cnt ? __builtin_nontemporal_load(pl.codes_b + bbase + r) : 0ull;
    }
    {
        typedef unsigned int v4u __attribute__((ext_vector_type(4)));
        for (int t = tid; t < nbk * kGroup; t += kBuildThreads) {
            const v4u x = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(gl) + t);
            tab[staged(t >> 3, t & 7)] = make_uint4(x.x, x.y, x.z, x.w);
        }
    }
    if (tid == 0) s_tombs = 0;
    __syncthreads();

    unsigned long long* tab64 = reinterpret_cast<unsigned long long*>(tab);
    const int32_t* tab32 = reinterpret_cast<const int32_t*>(tab);
    bool changed = false;
    for (int rb = 0; rb < cnt; rb += kBuildThreads * kBuildRecs) {
        if (rb > 0) {
#pragma unroll
            for (int k = 0; k < kBuildRecs; ++k) {
                const int r = rb + k * kBuildThreads + tid;
                codes[k] = r < cnt ? __builtin_nontemporal_load(pl.codes_b + bbase + r) : 0ull;
            }
        }
        int32_t freed[kBuildRecs];
        int ntomb = 0;
#pragma unroll
        for (int k = 0; k < kBuildRecs; ++k) {
            const int r = rb + k * kBuildThreads + tid;
            freed[k] = -1;
            if (r >= cnt) continue;
            const uint64_t code = codes[k];
            int lb = static_cast<int>(bucket_of(code, m.nb) - b0);
            for (int visited = 0; visited < nbk; ++visited) {
                int slot = -1;
                bool has_empty = false;
#pragma unroll
                for (int q = 0; q < kSlots / 2; ++q) {
                    const uint4 w = tab[staged(lb, q)];
                    const uint64_t c0 = static_cast<uint64_t>(w.x) | (static_cast<uint64_t>(w.y) << 32);
                    const uint64_t c1 = static_cast<uint64_t>(w.z) | (static_cast<uint64_t>(w.w) << 32);
                    if (c0 == code) slot = 2 * q;
                    if (c1 == code) slot = 2 * q + 1;
                    has_empty |= c0 == kEmpty || c1 == kEmpty;
                }
                if (slot >= 0) {
                    // the same key twice in the batch: one of the two frees it
                    const unsigned long long old = atomicCAS(
                            tab64 + staged(lb, slot >> 1) * 2 + (slot & 1), code,
                            has_empty ? kEmpty : kTomb);
                    if (old == code) {
                        freed[k] = tab32[staged(lb, (kValDword0 + slot) >> 2) * 4 + (slot & 3)];
                        ntomb += has_empty ? 0 : 1;
                    }
                    break;
                }
                if (has_empty) break;   // not stored
                if (++lb == nbk) lb = 0;
            }
        }
        if (ntomb) atomicAdd(&s_tombs, ntomb);
        int wrank[kBuildRecs];
#pragma unroll
        for (int k = 0; k < kBuildRecs; ++k) {
            const uint64_t wm = __ballot(freed[k] >= 0);
            wrank[k] = __popcll(wm & ((1ull << lane) - 1ull));
            if (lane == 0) s_wcnt[k * (kBuildThreads / 64) + wave] = __popcll(wm);
        }
        __syncthreads();
        if (tid == 0) {
            int tot = 0;
            for (int q = 0; q < kBuildRecs * (kBuildThreads / 64); ++q) {
                const int c = s_wcnt[q];
                s_wcnt[q] = tot;
                tot += c;
            }
            s_base = tot > 0 ? atomicSub(m.ctr + kCtrSize, tot) : 0;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < kBuildRecs; ++k) {
            if (freed[k] < 0) continue;
            changed = true;
            const int pos = s_base - 1 - (s_wcnt[k * (kBuildThreads / 64) + wave] + wrank[k]);
            if (pos >= 0 && pos < m.capacity) m.heap[pos] = freed[k];
            if (freed[k] < m.capacity) m.klog[freed[k]] = kEmpty;
        }
        __syncthreads();
    }
    if (!__syncthreads_or(changed ? 1 : 0)) return;
    {
        typedef unsigned int v4u __attribute__((ext_vector_type(4)));
        for (int t = tid; t < nbk * kGroup; t += kBuildThreads) {
            const uint4 x = tab[staged(t >> 3, t & 7)];
            const v4u y = {x.x, x.y, x.z, x.w};
            __builtin_nontemporal_store(y, reinterpret_cast<v4u*>(gl) + t);
        }
    }
    if (tid == 0 && s_tombs) atomicAdd(m.ctr + kCtrTombs, s_tombs);
}

// Provisional scheme, after the build pass: U = n - losers rows won a slot and
// the heap positions base .. base + U - 1 are the ones in use.  Thread t moves
// 32-bit word t of a value plane: row i = t / RD goes to the row of its
// promised position when i is a winner below U; with the heap in its initial
// order that is one contiguous copy.  RD = row width in words, 0 = read it from
// `rd` (widths 1..4 are compiled in so that the division is by a constant).
template <int RD>
__device__ __forceinline__ void copy_plane(const MapDev& m, const BulkPlan& pl,
                                           const uint32_t* __restrict__ src,
                                           uint32_t* __restrict__ dst, int rd_runtime,
                                           int64_t winners, int32_t heap_base, int identity) {
    const uint32_t rd = RD > 0 ? static_cast<uint32_t>(RD) : static_cast<uint32_t>(rd_runtime);
    const int64_t words = winners * rd;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kCopyThreads;
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * kCopyThreads + threadIdx.x;
    const bool narrow = words <= 0xFFFFFFFFll;   // the common case: 32-bit divisions
    auto row_of = [&](int64_t w) {
        return narrow ? static_cast<int64_t>(static_cast<uint32_t>(w) / rd) : w / rd;
    };
    auto move_word = [&](int64_t w) {
        const int64_t row = row_of(w);
        if (pl.flags[row] != 0) return;
        const uint32_t q = static_cast<uint32_t>(w - row * rd);
        const int64_t pos = heap_base + row;
        const int64_t idx = identity ? pos : m.heap[pos];
        dst[idx * rd + q] = src[w];
    };
    uint32_t* __restrict__ to = dst + static_cast<int64_t>(heap_base) * rd;
    const bool wide = identity && reinterpret_cast<uintptr_t>(src) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(to) % 16 == 0;
    if (!wide) {
        for (int64_t w = tid; w < words; w += stride) move_word(w);
        return;
    }
    // With the heap in its initial order the rows go to one contiguous range
    // that starts at `to`: 16 bytes per thread wherever none of the (up to four)
    // rows under them lost; the flags are not even read when no row lost.
    const bool clean = pl.hdr[kHdrLosers] == 0;
    const int64_t quads = words / 4;
    for (int64_t t = tid; t < quads; t += stride) {
        bool all = clean;
        if (!clean) {
            const int64_t lo = row_of(4 * t), hi = row_of(4 * t + 3);
            all = true;
            for (int64_t r = lo; r <= hi; ++r) all = all && pl.flags[r] == 0;
        }
        if (all) {
            {
                typedef unsigned int v4u __attribute__((ext_vector_type(4)));
                const v4u xl = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(src) + t);
                const uint4 x = make_uint4(xl.x, xl.y, xl.z, xl.w);
                v4u y = {x.x, x.y, x.z, x.w};
                __builtin_nontemporal_store(y, reinterpret_cast<v4u*>(to) + t);
            }
        } else {
            for (int q = 0; q < 4; ++q) move_word(4 * t + q);
        }
    }
    if (tid < words - 4 * quads) move_word(4 * quads + tid);
}

__global__ __launch_bounds__(kCopyThreads) void copy_rows_kernel(
        MapDev m, BulkPlan pl, ValueArgs va, int identity) {
    const int32_t heap_base = pl.hdr[kHdrBase];
    const int64_t winners = pl.n - pl.hdr[kHdrLosers];
    for (int v = 0; v < va.n; ++v) {
        const int rd = va.row_dwords[v];
        switch (rd) {
            case 1:
                copy_plane<1>(m, pl, va.src[v], va.dst[v], rd, winners, heap_base, identity);
                break;
            case 2:
                copy_plane<2>(m, pl, va.src[v], va.dst[v], rd, winners, heap_base, identity);
                break;
            case 3:
                copy_plane<3>(m, pl, va.src[v], va.dst[v], rd, winners, heap_base, identity);
                break;
            case 4:
                copy_plane<4>(m, pl, va.src[v], va.dst[v], rd, winners, heap_base, identity);
                break;
            default:
                copy_plane<0>(m, pl, va.src[v], va.dst[v], rd, winners, heap_base, identity);
                break;
        }
    }
}

// Positions of `mine` set lanes of the workgroup in a list that grows through
// the counter `cursor`: one update of the counter per workgroup (updates of a
// single address serialise across the device).  Every thread calls this; the
// return value is the caller's position (meaningful when `mine`).
constexpr int kListThreads = 1024;

__device__ __forceinline__ int reserve_in_list(bool mine, int32_t* cursor, int* s_wave,
                                               int* s_first) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const uint64_t mm = __ballot(mine);
    if (lane == 0) s_wave[wave] = __popcll(mm);
    __syncthreads();
    if (threadIdx.x == 0) {
        int tot = 0;
        for (int q = 0; q < kListThreads / 64; ++q) {
            const int c = s_wave[q];
            s_wave[q] = tot;
            tot += c;
        }
        *s_first = tot ? atomicAdd(cursor, tot) : 0;
    }
    __syncthreads();
    const int at = *s_first + s_wave[wave] + __popcll(mm & ((1ull << lane) - 1ull));
    __syncthreads();   // s_wave / s_first are reused by the next call
    return at;
}

// Provisional scheme, only when rows lost: the losers below row U are the
// holes that the winners at or beyond U move into.  Sixteen flags per thread;
// a workgroup that meets no loser (the usual case: a handful of rows lost among
// millions) goes on without touching the list.
__global__ __launch_bounds__(kListThreads) void list_holes_kernel(BulkPlan pl) {
    __shared__ int s_wave[kListThreads / 64];
    __shared__ int s_first;
    const int32_t losers = pl.hdr[kHdrLosers];
    if (losers == 0) return;
    const int64_t winners = pl.n - losers;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    for (int64_t first = static_cast<int64_t>(blockIdx.x) * kListThreads * 16; first < winners;
         first += static_cast<int64_t>(gridDim.x) * kListThreads * 16) {
        const int64_t i0 = first + static_cast<int64_t>(threadIdx.x) * 16;
        uint32_t w[4] = {0u, 0u, 0u, 0u};
        if (i0 + 16 <= winners) {
            // flags start 256-byte aligned and i0 is a multiple of 16
            const uint4 q = *reinterpret_cast<const uint4*>(pl.flags + i0);
            w[0] = q.x;
            w[1] = q.y;
            w[2] = q.z;
            w[3] = q.w;
        } else {
            for (int b = 0; b < 16 && i0 + b < winners; ++b) {
                w[b >> 2] |= static_cast<uint32_t>(pl.flags[i0 + b] != 0) << (8 * (b & 3));
            }
        }
        int cnt = 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            cnt += (w[q] & 0xFFu ? 1 : 0) + (w[q] & 0xFF00u ? 1 : 0) +
                   (w[q] & 0xFF0000u ? 1 : 0) + (w[q] & 0xFF000000u ? 1 : 0);
        }
        if (!__syncthreads_or(cnt)) continue;
        int incl = cnt;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(incl, d);
            if (lane >= d) incl += up;
        }
        if (lane == 63) s_wave[wave] = incl;
        __syncthreads();
        if (threadIdx.x == 0) {
            int tot = 0;
            for (int q = 0; q < kListThreads / 64; ++q) {
                const int c = s_wave[q];
                s_wave[q] = tot;
                tot += c;
            }
            s_first = atomicAdd(pl.hdr + kHdrHoles, tot);
        }
        __syncthreads();
        int at = s_first + s_wave[wave] + incl - cnt;
        for (int b = 0; b < 16 && cnt > 0; ++b) {
            if ((w[b >> 2] >> (8 * (b & 3))) & 0xFFu) {
                pl.holes[at++] = static_cast<int32_t>(i0 + b);
            }
        }
        __syncthreads();   // s_wave / s_first are reused by the next round
    }
}

// The slot that holds `code` (which is stored), by one lane on its own.
__device__ __forceinline__ int32_t* locate_index(const MapDev& m, uint64_t code) {
    uint32_t b = bucket_of(code, m.nb);
    for (uint32_t steps = 0; steps < kPartBuckets; ++steps) {
        const uint64_t* line = m.buckets + static_cast<size_t>(b) * kBucketQwords;
        for (int s = 0; s < kSlots; ++s) {
            if (line[s] == code) {
                return reinterpret_cast<int32_t*>(m.buckets) +
                       static_cast<size_t>(b) * kBucketDwords + kValDword0 + s;
            }
        }
        b = next_bucket(b, m.nb);
    }
    return nullptr;
}

// Provisional scheme, last step: sets the heap counter, and if rows lost,
// moves every winner at or beyond row U into a hole below U: its slot gets the
// index of the hole's position and its value rows are copied there.
template <int DIM>
__global__ __launch_bounds__(kListThreads) void settle_rows_kernel(
        MapDev m, BulkPlan pl, const int32_t* __restrict__ keys, ValueArgs va,
        int identity) {
    __shared__ int s_wave[kListThreads / 64];
    __shared__ int s_first;
    const int32_t heap_base = pl.hdr[kHdrBase];
    const int32_t losers = pl.hdr[kHdrLosers];
    const int64_t winners = pl.n - losers;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        m.ctr[kCtrSize] = heap_base + static_cast<int32_t>(winners);
    }
    if (losers == 0) return;
    const int64_t fit = rows_that_fit(m, pl);
    for (int64_t first = winners + static_cast<int64_t>(blockIdx.x) * kListThreads; first < fit;
         first += static_cast<int64_t>(gridDim.x) * kListThreads) {
        const int64_t i = first + threadIdx.x;
        const bool high = i < fit && pl.flags[i] == 0;
        const int at = reserve_in_list(high, pl.hdr + kHdrTaken, s_wave, &s_first);
        // positions from base + U on are free again: those of the rows that lost
        // (pass 1 has written their log entry when the heap is in its initial
        // order) and those that the high winners leave
        if (i < fit && (identity || high)) {
            const int64_t old_pos = heap_base + i;
            m.klog[identity ? old_pos : static_cast<int64_t>(m.heap[old_pos])] = kEmpty;
        }
        if (!high) continue;
        const int64_t pos = heap_base + pl.holes[at];
        const int32_t idx = identity ? static_cast<int32_t>(pos) : m.heap[pos];
        int32_t key[DIM];
        load_key<DIM>(keys, i, true, key);
        uint64_t code;
        pack_key<DIM>(key, code);
        int32_t* slot = locate_index(m, code);
        if (slot != nullptr) *slot = idx;
        m.klog[idx] = code;
        for (int v = 0; v < va.n; ++v) {
            const int rd = va.row_dwords[v];
            const uint32_t* s = va.src[v] + i * rd;
            uint32_t* d = va.dst[v] + static_cast<int64_t>(idx) * rd;
            for (int q = 0; q < rd; ++q) d[q] = s[q];
        }
    }
}

int check_values(int n_values, const void* const* src, void* const* dst,
                 const int64_t* row_bytes) {
    if (n_values < 0) ASH_FAIL("negative value count");
    if (n_values == 0) return 0;
    if (src == nullptr || dst == nullptr || row_bytes == nullptr) {
        ASH_FAIL("null value tables");
    }
    for (int v = 0; v < n_values; ++v) {
        if (src[v] == nullptr || dst[v] == nullptr) ASH_FAIL("null value tensor");
        if (row_bytes[v] <= 0) ASH_FAIL("value rows must not be empty");
    }
    return 0;
}

template <bool PROV>
int launch_split_keys(ash_map* map, const BulkPlan& pl, const int32_t* keys, int identity,
                      int32_t* early, hipStream_t s) {
    const unsigned g = static_cast<unsigned>((pl.n + kSplitChunk - 1) / kSplitChunk);
    switch (map->key_dim) {
        case 1:
            split_keys_kernel<1, PROV><<<g, kSplitThreads, 0, s>>>(map->d, pl, keys, identity, early);
            break;
        case 2:
            split_keys_kernel<2, PROV><<<g, kSplitThreads, 0, s>>>(map->d, pl, keys, identity, early);
            break;
        case 3:
            split_keys_kernel<3, PROV><<<g, kSplitThreads, 0, s>>>(map->d, pl, keys, identity, early);
            break;
        default:
            split_keys_kernel<4, PROV><<<g, kSplitThreads, 0, s>>>(map->d, pl, keys, identity, early);
            break;
    }
    ASH_LAUNCH_CHECK();
    return 0;
}

int launch_settle_rows(ash_map* map, const BulkPlan& pl, const int32_t* keys,
                       const ValueArgs& va, int identity, hipStream_t s) {
    // both leave at once when no row lost: grids that cost little to launch
    constexpr unsigned g = 128;
    list_holes_kernel<<<g, kListThreads, 0, s>>>(pl);
    ASH_LAUNCH_CHECK();
    switch (map->key_dim) {
        case 1:
            settle_rows_kernel<1><<<g, kListThreads, 0, s>>>(map->d, pl, keys, va, identity);
            break;
        case 2:
            settle_rows_kernel<2><<<g, kListThreads, 0, s>>>(map->d, pl, keys, va, identity);
            break;
        case 3:
            settle_rows_kernel<3><<<g, kListThreads, 0, s>>>(map->d, pl, keys, va, identity);
            break;
        default:
            settle_rows_kernel<4><<<g, kListThreads, 0, s>>>(map->d, pl, keys, va, identity);
            break;
    }
    ASH_LAUNCH_CHECK();
    return 0;
}

}  // namespace
}  // namespace ash

using namespace ash;

extern "C" {

int ash_map_bulk_workspace_bytes(ash_map_t* map, int64_t n, int n_values,
                                 const int64_t* row_bytes, int64_t* bytes,
                                 int* worthwhile) {
    if (map == nullptr) ASH_FAIL("null map handle");
    if (bytes == nullptr) ASH_FAIL("null output pointer");
    if (n_values > 0 && row_bytes == nullptr) ASH_FAIL("null value tables");
    BulkPlan pl;
    *bytes = make_plan(map, n, n_values, row_bytes, nullptr, pl);
    if (worthwhile) {
        // The build pass streams the whole table once, the per-key kernel costs
        // about as much per key as streaming three buckets.  Measured on
        // MI355X (16 M-slot table): keys only, the streaming path wins from
        // about one key per bucket; with value rows from about 1.5.
        // A table below 2^19 buckets has too few partitions to fill the device
        // in the build pass (a batch that large for it is mostly duplicates,
        // which the per-key kernel handles without atomics).
        const int64_t nb = static_cast<int64_t>(map->d.nb);
        bool big = nb >= (int64_t{1} << 19) &&
                   (n_values > 0 ? (n >= (int64_t{1} << 21) && 2 * n >= 3 * nb)
                                 : (n >= (int64_t{1} << 20) && n >= nb));
        // A table that was emptied (or made) and not used since still has to
        // be filled before the per-key kernel can run; the build pass writes
        // every range anyway and saves that fill.  Measured for such tables:
        // the streaming path wins from 2^18 keys and a third of a key per
        // bucket (half with value rows): 1 M keys into a new table of capacity
        // 2 M take 77 us instead of 138.  Not for batches far beyond what the
        // table holds (piles of duplicates would queue on a few ranges).
        if (map->table_stale && n >= (int64_t{1} << 18) && n <= 12 * nb &&
            (n_values > 0 ? 2 * n >= nb : 3 * n >= nb)) {
            big = true;
        }
        *worthwhile = (*bytes > 0 && big) ? 1 : 0;
    }
    return 0;
}

}  // extern "C"

// `early`: where to leave, right after the first split pass, the number of keys
// that pass handed to the per-key kernel; `early_event` is recorded behind it.
int ash::insert_bulk(ash_map* map, const int32_t* keys, int64_t n,
                     int n_values, const void* const* src, void* const* dst,
                     const int64_t* row_bytes, void* workspace,
                     int64_t workspace_bytes, int32_t* early, hipEvent_t early_event,
                     void* stream) {
    if (check_batch(map, keys, n)) return 1;
    if (check_values(n_values, src, dst, row_bytes)) return 1;
    if (workspace == nullptr) ASH_FAIL("null bulk workspace");
    if (reinterpret_cast<uintptr_t>(workspace) % 256 != 0) {
        ASH_FAIL("bulk workspace must be 256-byte aligned");
    }
    BulkPlan pl;
    const int64_t need = make_plan(map, n, n_values, row_bytes,
                                   static_cast<char*>(workspace), pl);
    if (need == 0) ASH_FAIL("the bulk path does not apply to this batch");
    if (workspace_bytes < need) ASH_FAIL("bulk workspace too small");
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (map->table_stale && is_capturing(s)) {
        // A cleared table whose fill is still pending is rewritten whole by the
        // build pass.  Captured into a graph that decision would be replayed
        // against whatever the table holds then.
        ASH_FAIL("the table was cleared and not used since: run one call outside the capture first");
    }

    ValueArgs user = {};
    user.n = n_values;
    for (int v = 0; v < n_values; ++v) {
        user.src[v] = static_cast<const uint32_t*>(src[v]);
        user.dst[v] = static_cast<uint32_t*>(dst[v]);
        user.row_dwords[v] = static_cast<int32_t>(row_bytes[v] / 4);
    }
    const ValueArgs none = {};
    const int stale = map->table_stale ? 1 : 0;
    counters_changed(map, true, s);
    // (captured into a graph, the choice would be replayed whatever the heap
    // holds then: a captured call takes the variant that reads the heap)
    const int identity = heap_in_order(map) ? 1 : 0;

    const int ncursors = static_cast<int>(pl.bins << pl.fine_shift);   // (>= bins << lane_shift)
    const int ninit = ncursors > kHdrWords ? ncursors : kHdrWords;
    bulk_init_kernel<<<(ninit + 255) / 256, 256, 0, s>>>(map->d, pl, ncursors);
    ASH_LAUNCH_CHECK();
    // (pass 1 leaves the early word itself; the event tells the host when)
    auto publish = [&]() -> int {
        if (early != nullptr && early_event != nullptr) ASH_HIP(hipEventRecord(early_event, s));
        return 0;
    };
    if (n_values == 0) {
        if (launch_split_keys<false>(map, pl, keys, identity, early, s)) return 1;
        if (publish()) return 1;
        split_records_kernel<false><<<(pl.bins << pl.lane_shift) * pl.chunks, kSplitThreads, 0, s>>>(map->d, pl);
        ASH_LAUNCH_CHECK();
        build_kernel<false><<<pl.parts, kBuildThreads, 0, s>>>(map->d, pl, stale, identity);
        ASH_LAUNCH_CHECK();
        map->table_stale = false;
        if (insert_selected(map, false, keys, pl.spill_keys, pl.hdr + kHdrSpillKeys, none, s)) {
            return 1;
        }
        return insert_selected(map, true, pl.codes_a, pl.spill_a, pl.hdr + kHdrSpillA, none, s);
    }
    if (launch_split_keys<true>(map, pl, keys, identity, early, s)) return 1;
    if (publish()) return 1;
    split_records_kernel<true><<<(pl.bins << pl.lane_shift) * pl.chunks, kSplitThreads, 0, s>>>(map->d, pl);
    ASH_LAUNCH_CHECK();
    build_kernel<true><<<pl.parts, kBuildThreads, 0, s>>>(map->d, pl, stale, identity);
    ASH_LAUNCH_CHECK();
    map->table_stale = false;
    int64_t words = 0;
    for (int v = 0; v < n_values; ++v) words = words > n * user.row_dwords[v] ? words : n * user.row_dwords[v];
    int64_t blocks = (words + kCopyThreads - 1) / kCopyThreads;
    if (blocks > 256 * 64) blocks = 256 * 64;
    copy_rows_kernel<<<static_cast<unsigned>(blocks), kCopyThreads, 0, s>>>(map->d, pl, user, identity);
    ASH_LAUNCH_CHECK();
    if (launch_settle_rows(map, pl, keys, user, identity, s)) return 1;
    return insert_selected(map, false, keys, pl.spill_keys, pl.hdr + kHdrSpillKeys, user, s);
}

extern "C" {

int ash_map_insert_bulk(ash_map_t* map, const int32_t* keys, int64_t n,
                        int n_values, const void* const* src, void* const* dst,
                        const int64_t* row_bytes, void* workspace,
                        int64_t workspace_bytes, void* stream) {
    return insert_bulk(map, keys, n, n_values, src, dst, row_bytes, workspace, workspace_bytes,
                       nullptr, nullptr, stream);
}

int ash_map_erase_bulk_query(ash_map_t* map, int64_t n, int64_t* bytes, int* worthwhile) {
    if (map == nullptr) ASH_FAIL("null map handle");
    if (bytes == nullptr) ASH_FAIL("null output pointer");
    BulkPlan pl;
    *bytes = make_plan(map, n, 0, nullptr, nullptr, pl);
    if (worthwhile) {
        // The range pass reads the whole table and writes back what changed; the
        // per-key kernel is bound by the device's atomic rate (19 G keys/s).
        // Measured on a 4 M-bucket table: 0.27 ms for the table plus 24 ps per
        // key against 53 ps per key, so the streaming path wins from about 2.3
        // keys per bucket.
        const int64_t nb = static_cast<int64_t>(map->d.nb);
        *worthwhile = (*bytes > 0 && nb >= (int64_t{1} << 19) && 2 * n >= 5 * nb) ? 1 : 0;
    }
    return 0;
}

int ash_map_erase_bulk(ash_map_t* map, const int32_t* keys, int64_t n, void* workspace,
                       int64_t workspace_bytes, void* stream) {
    if (check_batch(map, keys, n)) return 1;
    if (workspace == nullptr) ASH_FAIL("null bulk workspace");
    if (reinterpret_cast<uintptr_t>(workspace) % 256 != 0) {
        ASH_FAIL("bulk workspace must be 256-byte aligned");
    }
    BulkPlan pl;
    const int64_t need = make_plan(map, n, 0, nullptr, static_cast<char*>(workspace), pl);
    if (need == 0) ASH_FAIL("the bulk path does not apply to this batch");
    if (workspace_bytes < need) ASH_FAIL("bulk workspace too small");
    DeviceGuard guard;
    ASH_HIP(guard.enter(map->device));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (settle_table(map, s)) return 1;
    if (give_up_heap_order(map, s)) return 1;   // freed indices go back onto the heap
    counters_changed(map, false, s);
    const int ncursors = static_cast<int>(pl.bins << pl.fine_shift);   // (>= bins << lane_shift)
    const int ninit = ncursors > kHdrWords ? ncursors : kHdrWords;
    bulk_init_kernel<<<(ninit + 255) / 256, 256, 0, s>>>(map->d, pl, ncursors);
    ASH_LAUNCH_CHECK();
    if (launch_split_keys<false>(map, pl, keys, 0, nullptr, s)) return 1;
    split_records_kernel<false><<<(pl.bins << pl.lane_shift) * pl.chunks, kSplitThreads, 0, s>>>(map->d, pl);
    ASH_LAUNCH_CHECK();
    erase_range_kernel<<<pl.parts, kBuildThreads, 0, s>>>(map->d, pl);
    ASH_LAUNCH_CHECK();
    // keys that do not pack, and records beyond the capacity of a bin or range
    if (erase_selected(map, false, keys, pl.spill_keys, pl.hdr + kHdrSpillKeys, s)) return 1;
    return erase_selected(map, true, pl.codes_a, pl.spill_a, pl.hdr + kHdrSpillA, s);
}

}  // extern "C"
