// Bulk insert of libash_hip.so: builds the table in LDS instead of claiming
// slots with one global compare-and-swap per key.
//
// The per-key kernel (ash_map.hip) is bound by the rate at which the device
// executes atomics on random lines (about 2e10 per second, whatever cache the
// line sits in).  When a batch is of the order of the table itself it is
// cheaper to stream: the batch is split by bucket range in two coalesced
// passes (coarse bins, then partitions of 512 buckets inside each bin), and one
// workgroup per partition then owns 64 KB of the table exclusively: it loads
// that range into LDS (or starts from an empty one), inserts its records with
// LDS compare-and-swap, takes all indices of the partition from the heap with a
// single update of the heap counter, copies the value rows of the new keys and
// writes the range back with full-line stores.
//
// Records travel as a plane of 64-bit key codes plus one plane per value
// tensor, so every pass reads and writes contiguous runs.  Bins and partitions
// have a fixed capacity (expected count + ten standard deviations); what does
// not fit -- duplicates piled on one key, unpackable keys, a probe sequence
// that leaves its partition, an exhausted heap -- is put on a spill list and
// handled afterwards by the per-key kernel, so the result is the same map for
// any input.  The heap protocol is the reference's
// (ash/src/hashmap_gpu.cuh:211-232): a new key takes heap[counter++].
#include "ash_table.h"

#include "../../include/ash_hip.h"

#include <cmath>

namespace ash {
namespace {

constexpr int kPartShift = 9;
constexpr int kPartBuckets = 1 << kPartShift;   // buckets per build workgroup
// Chunk geometry measured on 16 M keys with two value planes (ms per insert):
// 1024x4 1.03, 1024x2 1.06, 512x4 1.13, 512x8 1.17, 256x8 1.29.
constexpr int kSplitThreads = 1024;
constexpr int kSplitKeys = 4;                   // records per thread
constexpr int kStageDwords = 4;                 // widest row slice staged in LDS
constexpr int kSplitChunk = kSplitThreads * kSplitKeys;
constexpr int kMaxBins = 256;
constexpr int kBuildThreads = 512;
constexpr int kBuildRecs = 4;                   // records per thread and round
constexpr int64_t kMinKeys = 1 << 12;

// Header words at the start of the workspace.
enum { kHdrSpillKeys = 0, kHdrSpillA = 1, kHdrSpillB = 2, kHdrWasEmpty = 3,
       kHdrWords = 64 };

struct BulkPlan {
    int64_t n;
    uint32_t parts;        // partitions of kPartBuckets buckets
    uint32_t bins;         // coarse bins of (1 << fine_shift) partitions
    uint32_t fine_shift;
    uint32_t cap_bin;      // records per coarse bin
    uint32_t cap_part;     // records per partition
    uint32_t chunks;       // split chunks per coarse bin
    int32_t* hdr;
    int32_t* cursor_bin;   // bins
    int32_t* cursor_part;  // bins << fine_shift
    uint64_t* codes_a;     // bins * cap_bin
    uint64_t* codes_b;     // parts * cap_part
    uint32_t* plane_a[kMaxFusedValues];
    uint32_t* plane_b[kMaxFusedValues];
    int32_t* spill_keys;   // n input row numbers
    int32_t* spill_a;      // n positions in the coarse planes
    int32_t* spill_b;      // n positions in the partition planes
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
    const double mean_bin = per_bucket * kPartBuckets * static_cast<double>(1ll << fine_shift);
    const double mean_part = per_bucket * kPartBuckets;
    int64_t cap_bin = static_cast<int64_t>(mean_bin + 10.0 * std::sqrt(mean_bin)) + 256;
    int64_t cap_part = static_cast<int64_t>(mean_part + 10.0 * std::sqrt(mean_part)) + 64;
    if (cap_bin > n) cap_bin = n;
    if (cap_part > n) cap_part = n;
    cap_bin = (cap_bin + 15) & ~int64_t{15};
    cap_part = (cap_part + 15) & ~int64_t{15};
    const int64_t na = bins * cap_bin;
    const int64_t nbp = parts * cap_part;
    if (na >= (int64_t{1} << 31) || nbp >= (int64_t{1} << 31)) return 0;

    pl.n = n;
    pl.parts = static_cast<uint32_t>(parts);
    pl.bins = static_cast<uint32_t>(bins);
    pl.fine_shift = fine_shift;
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
    pl.cursor_bin = reinterpret_cast<int32_t*>(take(bins * 4));
    pl.cursor_part = reinterpret_cast<int32_t*>(take((bins << fine_shift) * 4));
    pl.codes_a = reinterpret_cast<uint64_t*>(take(na * 8));
    pl.codes_b = reinterpret_cast<uint64_t*>(take(nbp * 8));
    for (int v = 0; v < kMaxFusedValues; ++v) {
        pl.plane_a[v] = nullptr;
        pl.plane_b[v] = nullptr;
        if (v < n_values) {
            pl.plane_a[v] = reinterpret_cast<uint32_t*>(take(na * row_bytes[v]));
            pl.plane_b[v] = reinterpret_cast<uint32_t*>(take(nbp * row_bytes[v]));
        }
    }
    pl.spill_keys = reinterpret_cast<int32_t*>(take(n * 4));
    pl.spill_a = reinterpret_cast<int32_t*>(take(n * 4));
    pl.spill_b = reinterpret_cast<int32_t*>(take(n * 4));
    return off;
}

// ------------------------------------------------------------- kernels
__global__ void bulk_init_kernel(MapDev m, BulkPlan pl, int ncursors) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    // cursor_bin and cursor_part are zeroed separately: they are not adjacent
    if (t < static_cast<int>(pl.bins)) pl.cursor_bin[t] = 0;
    if (t < ncursors) pl.cursor_part[t] = 0;
    if (t == 0) {
        pl.hdr[kHdrSpillKeys] = 0;
        pl.hdr[kHdrSpillA] = 0;
        pl.hdr[kHdrSpillB] = 0;
        pl.hdr[kHdrWasEmpty] =
                (m.ctr[kCtrSize] == 0 && m.ctr[kCtrTombs] == 0) ? 1 : 0;
    }
}

__device__ __forceinline__ void copy_row(const uint32_t* __restrict__ s,
                                         uint32_t* __restrict__ d, int rd) {
    for (int q = 0; q < rd; ++q) d[q] = s[q];
}

// LDS of the two split passes.  Every record of the workgroup's chunk gets a
// bin and its arrival rank inside that bin (LDS counter); reserve_runs turns
// the counts into start[b] (first sorted position of bin b inside the chunk)
// and base[b] (position of the chunk's run inside the bin's global buffer,
// reserved with one atomic per bin).  The chunk is then moved plane by plane:
// each thread drops its records at their sorted positions in `stage`, and the
// workgroup writes the stage out front to back, so that global reads and
// writes both have consecutive lanes on consecutive records.
struct SplitShared {
    int cnt[kMaxBins];
    int start[kMaxBins];
    int base[kMaxBins];
    int wave_total[kMaxBins / 64];
    uint16_t perm[kSplitChunk];    // sorted position -> record of the chunk
    uint8_t bin_of[kSplitChunk];   // sorted position -> bin
    uint32_t stage[kSplitChunk * kStageDwords];
};

__device__ __forceinline__ int reserve_runs(SplitShared& sh, int32_t* cursors,
                                            int nbins) {
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
        sh.base[tid] = (v && tid < nbins) ? atomicAdd(cursors + tid, v) : 0;
    }
    __syncthreads();
    int total = 0;
#pragma unroll
    for (int w = 0; w < kMaxBins / 64; ++w) total += sh.wave_total[w];
    return total;
}

// Moves the ranked records of a chunk to their runs.  code/bin/rank describe
// the calling thread's kSplitKeys records (record k of the thread is record
// k * kSplitThreads + tid of the chunk, bin < 0 = not taking part); the value
// rows of record r are row `row0 + r` of src[v].  Destination of a record with
// bin b and position pos inside the bin: dst_first(b) + pos, valid while
// pos < cap; the others are reported through `spill` with their record number.
template <typename DstFirst, typename Spill>
__device__ __forceinline__ void move_chunk(
        SplitShared& sh, int total, const uint64_t (&code)[kSplitKeys],
        const int (&bin)[kSplitKeys], const int (&rank)[kSplitKeys],
        int64_t row0, const uint32_t* const (&src)[kMaxFusedValues],
        uint32_t* const (&dst)[kMaxFusedValues],
        const int32_t (&row_dwords)[kMaxFusedValues], int n_values,
        uint64_t* __restrict__ codes_dst, uint32_t cap, DstFirst dst_first,
        Spill spill) {
    const int tid = threadIdx.x;
    uint32_t regs[kSplitKeys][kStageDwords];
    auto load_slice = [&](int v, int q0) {
        const int rd = row_dwords[v];
        const int w = rd - q0 < kStageDwords ? rd - q0 : kStageDwords;
#pragma unroll
        for (int k = 0; k < kSplitKeys; ++k) {
            if (bin[k] >= 0) {
                const uint32_t* s =
                        src[v] + (row0 + k * kSplitThreads + tid) * rd + q0;
#pragma unroll
                for (int q = 0; q < kStageDwords; ++q) {
                    if (q < w) regs[k][q] = s[q];
                }
            }
        }
    };
    int v = 0, q0 = 0;
    bool have = n_values > 0;
    if (have) load_slice(0, 0);
    int sp[kSplitKeys];
#pragma unroll
    for (int k = 0; k < kSplitKeys; ++k) {
        sp[k] = -1;
        if (bin[k] >= 0) {
            sp[k] = sh.start[bin[k]] + rank[k];
            sh.perm[sp[k]] = static_cast<uint16_t>(k * kSplitThreads + tid);
            sh.bin_of[sp[k]] = static_cast<uint8_t>(bin[k]);
            reinterpret_cast<uint64_t*>(sh.stage)[sp[k]] = code[k];
        }
    }
    __syncthreads();
    int64_t d[kSplitKeys];
#pragma unroll
    for (int j = 0; j < kSplitKeys; ++j) {
        const int s = j * kSplitThreads + tid;
        d[j] = -1;
        if (s < total) {
            const int b = sh.bin_of[s];
            const uint32_t pos =
                    static_cast<uint32_t>(sh.base[b] + (s - sh.start[b]));
            if (pos < cap) {
                d[j] = dst_first(b) + pos;
                codes_dst[d[j]] = reinterpret_cast<const uint64_t*>(sh.stage)[s];
            } else {
                spill(static_cast<int>(sh.perm[s]));
            }
        }
    }
    // Value rows, one slice of up to kStageDwords words at a time.  The rows of
    // the next slice are requested while the current one is written out.
    while (have) {
        const int rd = row_dwords[v];
        const int w = rd - q0 < kStageDwords ? rd - q0 : kStageDwords;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < kSplitKeys; ++k) {
            if (sp[k] >= 0) {
#pragma unroll
                for (int q = 0; q < kStageDwords; ++q) {
                    if (q < w) sh.stage[sp[k] * w + q] = regs[k][q];
                }
            }
        }
        int nv = v, nq0 = q0 + kStageDwords;
        if (nq0 >= rd) {
            ++nv;
            nq0 = 0;
        }
        const bool nhave = nv < n_values;
        if (nhave) load_slice(nv, nq0);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < kSplitKeys; ++j) {
            if (d[j] >= 0) {
                const int s = j * kSplitThreads + tid;
                uint32_t* o = dst[v] + d[j] * rd + q0;
                for (int q = 0; q < w; ++q) o[q] = sh.stage[s * w + q];
            }
        }
        v = nv;
        q0 = nq0;
        have = nhave;
    }
}

// Pass 1: input rows -> coarse bins, 4096 keys per workgroup.
template <int DIM>
__global__ __launch_bounds__(kSplitThreads) void split_keys_kernel(
        MapDev m, BulkPlan pl, const int32_t* __restrict__ keys, ValueArgs va) {
    __shared__ SplitShared sh;
    const int tid = threadIdx.x;
    if (tid < kMaxBins) sh.cnt[tid] = 0;
    __syncthreads();
    const int64_t base = static_cast<int64_t>(blockIdx.x) * kSplitChunk;
    const int bin_shift = kPartShift + static_cast<int>(pl.fine_shift);
    uint64_t code[kSplitKeys];
    int bin[kSplitKeys];
    int rank[kSplitKeys];
#pragma unroll
    for (int k = 0; k < kSplitKeys; ++k) {
        const int64_t i = base + k * kSplitThreads + tid;
        const bool active = i < pl.n;
        int32_t key[DIM];
        load_key<DIM>(keys, i, active, key);
        const bool fits = pack_key<DIM>(key, code[k]);
        bin[k] = -1;
        rank[k] = 0;
        if (active && fits) {
            bin[k] = static_cast<int>(bucket_of(code[k], m.nb) >> bin_shift);
            rank[k] = atomicAdd(&sh.cnt[bin[k]], 1);
        } else if (active) {
            // unpackable: left to the per-key kernel
            pl.spill_keys[atomicAdd(pl.hdr + kHdrSpillKeys, 1)] =
                    static_cast<int32_t>(i);
        }
    }
    __syncthreads();
    const int total = reserve_runs(sh, pl.cursor_bin, static_cast<int>(pl.bins));
    move_chunk(
            sh, total, code, bin, rank, base, va.src, pl.plane_a, va.row_dwords,
            va.n, pl.codes_a, pl.cap_bin,
            [&](int b) { return static_cast<int64_t>(b) * pl.cap_bin; },
            [&](int rec) {
                pl.spill_keys[atomicAdd(pl.hdr + kHdrSpillKeys, 1)] =
                        static_cast<int32_t>(base + rec);
            });
}

// Pass 2: coarse bin -> partitions.  Workgroup (bin, chunk) takes 4096 records
// of its bin.
__global__ __launch_bounds__(kSplitThreads) void split_records_kernel(
        MapDev m, BulkPlan pl, ValueArgs va) {
    __shared__ SplitShared sh;
    const int tid = threadIdx.x;
    const uint32_t c = blockIdx.x / pl.chunks;
    const uint32_t chunk = blockIdx.x % pl.chunks;
    int cnt = pl.cursor_bin[c];
    if (cnt > static_cast<int>(pl.cap_bin)) cnt = static_cast<int>(pl.cap_bin);
    const int start = static_cast<int>(chunk) * kSplitChunk;
    if (start >= cnt) return;
    if (tid < kMaxBins) sh.cnt[tid] = 0;
    __syncthreads();
    const int64_t abase = static_cast<int64_t>(c) * pl.cap_bin + start;
    const uint32_t fmask = (1u << pl.fine_shift) - 1u;
    uint64_t code[kSplitKeys];
    int bin[kSplitKeys];
    int rank[kSplitKeys];
#pragma unroll
    for (int k = 0; k < kSplitKeys; ++k) {
        const int j = k * kSplitThreads + tid;
        bin[k] = -1;
        rank[k] = 0;
        code[k] = 0;
        if (start + j < cnt) {
            code[k] = pl.codes_a[abase + j];
            bin[k] = static_cast<int>((bucket_of(code[k], m.nb) >> kPartShift) & fmask);
            rank[k] = atomicAdd(&sh.cnt[bin[k]], 1);
        }
    }
    __syncthreads();
    const int total = reserve_runs(
            sh, pl.cursor_part + (static_cast<size_t>(c) << pl.fine_shift),
            static_cast<int>(fmask) + 1);
    const uint32_t* src[kMaxFusedValues];
#pragma unroll
    for (int v = 0; v < kMaxFusedValues; ++v) src[v] = pl.plane_a[v];
    move_chunk(
            sh, total, code, bin, rank, abase, src, pl.plane_b, va.row_dwords,
            va.n, pl.codes_b, pl.cap_part,
            [&](int b) {
                return static_cast<int64_t>((c << pl.fine_shift) +
                                            static_cast<uint32_t>(b)) *
                       pl.cap_part;
            },
            [&](int rec) {
                pl.spill_a[atomicAdd(pl.hdr + kHdrSpillA, 1)] =
                        static_cast<int32_t>(abase + rec);
            });
}

// Where the q-th 16 bytes of local bucket lb sit in the LDS copy of the table
// range.  A bucket is 128 bytes = 32 banks wide, so without the rotation every
// lane that reads "16 bytes number q of its bucket" would hit the same four
// banks; rotating by the bucket number spreads them over all of them.
__device__ __forceinline__ int staged(int lb, int q) {
    return lb * kGroup + ((q + lb) & (kGroup - 1));
}

// Pass 3: one workgroup per partition builds its 512 buckets in LDS.
// `stale`: the bucket array holds leftovers of a table that has been cleared
// since (the clear left the fill to its successor): every partition is then
// written, those without records as empty ones.
__global__ __launch_bounds__(kBuildThreads) void build_kernel(
        MapDev m, BulkPlan pl, ValueArgs va, int stale) {
    __shared__ uint4 tab[kPartBuckets * kGroup];
    // winners per (record slot k, wavefront), then their exclusive prefix
    __shared__ int s_wcnt[kBuildRecs * (kBuildThreads / 64)];
    __shared__ int s_base;
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
    const int64_t bbase = static_cast<int64_t>(p) * pl.cap_part;
    // The first round's records are requested before the table range is
    // staged, so that both latencies overlap.
    uint64_t codes[kBuildRecs];
#pragma unroll
    for (int k = 0; k < kBuildRecs; ++k) {
        const int r = k * kBuildThreads + tid;
        codes[k] = r < cnt ? pl.codes_b[bbase + r] : 0ull;
    }
    for (int t = tid; t < nbk * kGroup; t += kBuildThreads) {
        tab[staged(t >> 3, t & 7)] =
                was_empty ? make_uint4(~0u, ~0u, ~0u, ~0u) : gl[t];
    }
    __syncthreads();

    unsigned long long* tab64 = reinterpret_cast<unsigned long long*>(tab);
    int32_t* tab32 = reinterpret_cast<int32_t*>(tab);

    for (int rb = 0; rb < cnt; rb += kBuildThreads * kBuildRecs) {
        int wslot[kBuildRecs];
        int wrank[kBuildRecs];
        if (rb > 0) {
#pragma unroll
            for (int k = 0; k < kBuildRecs; ++k) {
                const int r = rb + k * kBuildThreads + tid;
                codes[k] = r < cnt ? pl.codes_b[bbase + r] : 0ull;
            }
        }
#pragma unroll
        for (int k = 0; k < kBuildRecs; ++k) {
            const int r = rb + k * kBuildThreads + tid;
            wslot[k] = -1;
            if (r >= cnt) continue;
            const uint64_t code = codes[k];

            int lb = static_cast<int>(bucket_of(code, m.nb) - b0);
            for (;;) {
                uint64_t c[kSlots];
#pragma unroll
                for (int q = 0; q < kSlots / 2; ++q) {
                    const uint4 w = tab[staged(lb, q)];
                    c[2 * q] = static_cast<uint64_t>(w.x) |
                               (static_cast<uint64_t>(w.y) << 32);
                    c[2 * q + 1] = static_cast<uint64_t>(w.z) |
                                   (static_cast<uint64_t>(w.w) << 32);
                }
                bool done = false;
                uint32_t em = 0;
#pragma unroll
                for (int s = 0; s < kSlots; ++s) {
                    done |= c[s] == code;
                    em |= (c[s] == kEmpty ? 1u : 0u) << s;
                }
                while (!done && em) {
                    const int s = __builtin_ctz(em);
                    const unsigned long long old =
                            atomicCAS(tab64 + staged(lb, s >> 1) * 2 + (s & 1),
                                      kEmpty, code);
                    if (old == kEmpty) {
                        wslot[k] = lb * kBucketQwords + s;
                        done = true;
                    } else if (old == code) {
                        done = true;
                    }
                    em &= em - 1;
                }
                if (done) break;
                if (++lb == nbk) {
                    // The probe sequence leaves this partition.
                    pl.spill_b[atomicAdd(pl.hdr + kHdrSpillB, 1)] =
                            static_cast<int32_t>(bbase + r);
                    break;
                }
            }
        }
        // Winners are ranked in record order, so that consecutive lanes take
        // consecutive heap entries and their value rows land side by side.
#pragma unroll
        for (int k = 0; k < kBuildRecs; ++k) {
            const uint64_t wm = __ballot(wslot[k] >= 0);
            wrank[k] = __popcll(wm & ((1ull << lane) - 1ull));
            if (lane == 0) s_wcnt[k * (kBuildThreads / 64) + wave] = __popcll(wm);
        }
        // The first slice of the winners' value rows does not depend on the
        // indices: it is requested now and travels while the heap counter and
        // the heap entries are fetched.
        uint32_t rows[kBuildRecs][kStageDwords];
        auto load_rows = [&](int v, int q0) {
            const int rd = va.row_dwords[v];
            const int w = rd - q0 < kStageDwords ? rd - q0 : kStageDwords;
#pragma unroll
            for (int k = 0; k < kBuildRecs; ++k) {
                if (wslot[k] >= 0) {
                    const uint32_t* s = pl.plane_b[v] +
                            (bbase + rb + k * kBuildThreads + tid) * rd + q0;
#pragma unroll
                    for (int q = 0; q < kStageDwords; ++q) {
                        if (q < w) rows[k][q] = s[q];
                    }
                }
            }
        };
        if (va.n > 0) load_rows(0, 0);
        __syncthreads();
        if (tid == 0) {
            int tot = 0;
            for (int q = 0; q < kBuildRecs * (kBuildThreads / 64); ++q) {
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
        int32_t idx[kBuildRecs];
#pragma unroll
        for (int k = 0; k < kBuildRecs; ++k) {
            idx[k] = -1;
            if (wslot[k] < 0) continue;
            const int top = s_base + s_wcnt[k * (kBuildThreads / 64) + wave] + wrank[k];
            if (top < m.capacity) {
                idx[k] = m.heap[top];
            } else {
                // Heap exhausted: give the slot up again.
                const int wlb = wslot[k] >> 4;
                const int ws = wslot[k] & 15;
                tab64[staged(wlb, ws >> 1) * 2 + (ws & 1)] = kTomb;
                atomicAdd(m.ctr + kCtrTombs, 1);
                wslot[k] = -1;
            }
        }
#pragma unroll
        for (int k = 0; k < kBuildRecs; ++k) {
            if (idx[k] >= 0) {
                const int wlb = wslot[k] >> 4;
                const int ws = wslot[k] & 15;
                tab32[staged(wlb, (kValDword0 + ws) >> 2) * 4 + (ws & 3)] = idx[k];
            }
        }
        for (int v = 0; v < va.n; ++v) {
            const int rd = va.row_dwords[v];
            for (int q0 = 0; q0 < rd; q0 += kStageDwords) {
                const int w = rd - q0 < kStageDwords ? rd - q0 : kStageDwords;
                if (v > 0 || q0 > 0) load_rows(v, q0);
#pragma unroll
                for (int k = 0; k < kBuildRecs; ++k) {
                    if (idx[k] >= 0) {
                        uint32_t* o = va.dst[v] + static_cast<int64_t>(idx[k]) * rd + q0;
#pragma unroll
                        for (int q = 0; q < kStageDwords; ++q) {
                            if (q < w) o[q] = rows[k][q];
                        }
                    }
                }
            }
        }
        __syncthreads();
    }
    for (int t = tid; t < nbk * kGroup; t += kBuildThreads) {
        gl[t] = tab[staged(t >> 3, t & 7)];
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
        // about one key per bucket; with value rows, which travel through both
        // split passes, from about 1.5.
        // A table below 2^19 buckets has too few partitions to fill the device
        // in the build pass (a batch that large for it is mostly duplicates,
        // which the per-key kernel handles without atomics).
        const int64_t nb = static_cast<int64_t>(map->d.nb);
        const bool big = nb >= (int64_t{1} << 19) &&
                         (n_values > 0 ? (n >= (int64_t{1} << 21) && 2 * n >= 3 * nb)
                                       : (n >= (int64_t{1} << 20) && n >= nb));
        *worthwhile = (*bytes > 0 && big) ? 1 : 0;
    }
    return 0;
}

int ash_map_insert_bulk(ash_map_t* map, const int32_t* keys, int64_t n,
                        int n_values, const void* const* src, void* const* dst,
                        const int64_t* row_bytes, void* workspace,
                        int64_t workspace_bytes, void* stream) {
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

    ValueArgs user = {};
    ValueArgs from_a = {};
    ValueArgs from_b = {};
    user.n = from_a.n = from_b.n = n_values;
    for (int v = 0; v < n_values; ++v) {
        const int32_t rd = static_cast<int32_t>(row_bytes[v] / 4);
        user.src[v] = static_cast<const uint32_t*>(src[v]);
        from_a.src[v] = pl.plane_a[v];
        from_b.src[v] = pl.plane_b[v];
        user.dst[v] = from_a.dst[v] = from_b.dst[v] = static_cast<uint32_t*>(dst[v]);
        user.row_dwords[v] = from_a.row_dwords[v] = from_b.row_dwords[v] = rd;
    }

    const int ncursors = static_cast<int>(pl.bins << pl.fine_shift);
    bulk_init_kernel<<<(ncursors + 255) / 256, 256, 0, s>>>(map->d, pl, ncursors);
    ASH_LAUNCH_CHECK();
    const unsigned g1 = static_cast<unsigned>((n + kSplitChunk - 1) / kSplitChunk);
    switch (map->key_dim) {
        case 1:
            split_keys_kernel<1><<<g1, kSplitThreads, 0, s>>>(map->d, pl, keys, user);
            break;
        case 2:
            split_keys_kernel<2><<<g1, kSplitThreads, 0, s>>>(map->d, pl, keys, user);
            break;
        case 3:
            split_keys_kernel<3><<<g1, kSplitThreads, 0, s>>>(map->d, pl, keys, user);
            break;
        default:
            split_keys_kernel<4><<<g1, kSplitThreads, 0, s>>>(map->d, pl, keys, user);
            break;
    }
    ASH_LAUNCH_CHECK();
    split_records_kernel<<<pl.bins * pl.chunks, kSplitThreads, 0, s>>>(map->d, pl,
                                                                      user);
    ASH_LAUNCH_CHECK();
    // A cleared table whose fill is still pending is empty by its counters, so
    // the build starts every partition from scratch and writes all of them.
    build_kernel<<<pl.parts, kBuildThreads, 0, s>>>(map->d, pl, from_b,
                                                    map->table_stale ? 1 : 0);
    ASH_LAUNCH_CHECK();
    map->table_stale = false;
    if (insert_selected(map, false, keys, pl.spill_keys, pl.hdr + kHdrSpillKeys,
                        user, s)) {
        return 1;
    }
    if (insert_selected(map, true, pl.codes_a, pl.spill_a, pl.hdr + kHdrSpillA,
                        from_a, s)) {
        return 1;
    }
    return insert_selected(map, true, pl.codes_b, pl.spill_b,
                           pl.hdr + kHdrSpillB, from_b, s);
}

}  // extern "C"
