// Shared host/device definitions for libash_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

namespace ash {

// ---------------------------------------------------------------- errors
void set_error(const std::string& msg);

#define ASH_FAIL(msg)                 \
    do {                              \
        ::ash::set_error(msg);        \
        return 1;                     \
    } while (0)

#define ASH_HIP(expr)                                                        \
    do {                                                                     \
        hipError_t _e = (expr);                                              \
        if (_e != hipSuccess) {                                              \
            ::ash::set_error(std::string(#expr) + ": " +                     \
                             hipGetErrorString(_e));                         \
            return 1;                                                        \
        }                                                                    \
    } while (0)

#define ASH_LAUNCH_CHECK() ASH_HIP(hipGetLastError())

// ------------------------------------------------------- table geometry
// One bucket is one 128-byte line read by a group of 8 lanes, 16 bytes each:
//   dwords [ 0,20)  ten 64-bit packed key codes
//   dwords [20,30)  ten int32 indices (slot s -> dword 20+s)
//   dwords [30,32)  unused
constexpr int kGroup = 8;                       // lanes per bucket
constexpr int kBucketDwords = kGroup * 4;       // 32
constexpr int kBucketQwords = kGroup * 2;       // 16
constexpr int kSlots = (kGroup * 16) / 12;      // 10
constexpr int kValDword0 = 2 * kSlots;          // 20
constexpr int kTargetFill = 6;                  // entries per bucket at capacity

constexpr uint64_t kEmpty = ~0ull;
constexpr uint64_t kTomb = ~0ull - 1ull;

// A probe sequence never leaves the aligned range of 512 buckets (64 KB) that
// the key's hash names: from the range's last bucket it goes on at its first.
// The streaming insert builds one such range per workgroup in LDS, and a range
// is what a key's neighbours in the table share in the caches.  At the table's
// load (six entries per ten-slot bucket at capacity) a range that is full is
// out of reach (its 5120 slots against a mean of at most 3072 entries with a
// standard deviation of 55; every range of a table with several is a whole
// one, see num_buckets); a key that finds its range full is refused and
// counted like a key that finds the heap exhausted.
constexpr int kPartShift = 9;
constexpr uint32_t kPartBuckets = 1u << kPartShift;

// Device counters kept in the first 256 bytes of the table workspace.
enum Counter {
    kCtrSize = 0,      // heap counter == number of live entries
    kCtrDropped = 1,   // keys refused because the heap was exhausted
    kCtrTombs = 2,     // tombstoned slots (packed + general)
    kCtrExotic = 3,    // unpackable keys seen while no general region exists
    kCtrLoadDup = 4,   // pairs refused by load: duplicate keys, indices outside 0 .. capacity-1
    kCtrGenLive = 5,   // entries that live in the general region
    kCtrTouched = 6,   // blocks listed by the latest ash_grid_collect_touched
    kCtrGenTombs = 7,  // of kCtrTombs, those in the general region
    // (the first eight are what a read-back of the counters copies to the host)
    kCtrLogHigh = 8,   // log entries at or beyond the size and below this index may hold keys of an earlier filling
    kCtrCursor = 9,    // output cursor of items()
    kCtrTicket = 10,   // workgroups of a running ash_grid_collect_touched that have read their input
    kNumCounters = 64
};
constexpr int kHostCounters = 8;
constexpr int64_t kHeaderBytes = 256;

// General region: open addressing over 32-bit state words + 16-byte keys.
constexpr int32_t kGenEmpty = -1;
constexpr int32_t kGenLocked = -2;
constexpr int32_t kGenTomb = -3;
constexpr int32_t kGenNoIndex = -4;  // key visible, index not yet assigned

struct MapDev {
    uint64_t* buckets;   // nb * 16 qwords
    // key log: klog[index] = packed code of the key stored under `index`,
    // kTomb when that key lives in the general region, kEmpty when the index
    // is free.  items() enumerates from here (8 bytes per index instead of the
    // whole bucket array) and therefore in index order, which is the order of
    // the callers' value rows.
    uint64_t* klog;      // capacity qwords
    int32_t* ctr;        // kNumCounters int32
    int32_t* heap;       // capacity int32 (caller-owned)
    int32_t* gstate;     // general region state/index words (or nullptr)
    int32_t* gkeys;      // general region keys, 4 int32 per slot
    uint32_t nb;         // number of buckets
    uint32_t gslots;     // general slots (power of two) or 0
    int32_t capacity;
};

// A table of more than one probe range consists of whole ranges: a short last
// range would receive a full bucket's share of the keys per bucket like every
// other and, having few slots, could fill up (and refuse keys) while the heap
// still has indices.  A table of at most kPartBuckets buckets is one range.
inline int64_t num_buckets(int64_t capacity) {
    int64_t nb = (capacity + kTargetFill - 1) / kTargetFill;
    if (nb < 2) nb = 2;
    if (nb > static_cast<int64_t>(kPartBuckets)) {
        nb = (nb + kPartBuckets - 1) & ~static_cast<int64_t>(kPartBuckets - 1);
    }
    return nb;
}

// Byte offset of the key log inside the table workspace.
inline int64_t klog_offset(int64_t capacity) {
    const int64_t end = kHeaderBytes + num_buckets(capacity) * kBucketDwords * 4;
    return (end + 255) & ~int64_t{255};
}

inline int64_t table_workspace_bytes(int64_t capacity) {
    // whole 16-byte units: the log is cleared and read two entries at a time
    return klog_offset(capacity) + ((capacity + 1) / 2) * 16;
}

// Slots of a general region that can hold `capacity` keys at half load; a
// caller may attach a smaller one (a power of two, at least kMinGeneralSlots).
constexpr int64_t kMinGeneralSlots = 64;
inline int64_t general_slots(int64_t capacity) {
    int64_t s = kMinGeneralSlots;
    while (s < 2 * capacity) s <<= 1;
    return s;
}

}  // namespace ash

// What the host knows of the device counters (ash_map_counters).
struct ash_counters {
    int64_t size, dropped, tombstones, exotic_pending, load_refused, touched, general_live,
            general_tombstones;
};

struct ash_map {
    int key_dim;
    int64_t capacity;
    int device;
    ash::MapDev d;
    int64_t table_bytes;
    bool general_attached;
    // --- bookkeeping of the counters on the host ------------------------
    // page-locked int32[16] of the caller's (ash_map_set_staging) or null:
    // [0, 8) landing place of a read-back, [8] the count a streaming insert
    // publishes after its first pass
    int32_t* staging;
    hipEvent_t early_event, late_event;   // made on first use
    bool late_in_flight;    // a copy into staging[0, 8) may still be under way
    bool late_pending;      // ... and it is the latest state of the counters: nobody has looked at it yet
    bool counters_known;    // `counters` is what the device holds
    ash_counters counters;
    // an erase, refused keys or a run of inserts whose counters nobody read
    // may have left tombstones: the next managed insert looks at the counters
    bool maybe_tombstones;
    int unread_inserts;
    // A call that changes the map has been captured into a graph: replays
    // change the device's state behind the host's back, so from then on nothing
    // the host remembers of it is trusted -- the counters are copied from the
    // device whenever they are asked for, the heap is read (never assumed to be
    // 0, 1, 2, ...), listings go by ranks and a clear clears at once.
    bool replayed;
    // clear() has reset the counters and the heap but left the bucket array as
    // it was: the next call that reads the table fills it first, a streaming
    // insert that rewrites every bucket does not need to
    bool table_stale;
    // the heap array may differ from 0, 1, 2, ... (an erase or a load has
    // written to it since it was last reset): clear() rewrites it only then
    bool heap_dirty;
    // a clear() has left the key log as it was (while the heap is in its
    // initial order only entries below the size are read): entries between
    // the size and the counter kCtrLogHigh are emptied before the order of
    // the heap is given up (give_up_heap_order)
    bool log_stale;
};
