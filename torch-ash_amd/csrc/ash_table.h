// Device-side helpers shared by the table kernels of libash_hip.so: key codec,
// hash, bucket addressing, the value-row descriptor of a fused insert.
#pragma once

#include "ash_dev.h"

namespace ash {

constexpr int kMaxFusedValues = 4;
constexpr int kMaxFusedRowDwords = 16;

// ------------------------------------------------------------ key codec
template <int DIM>
__device__ __forceinline__ bool pack_key(const int32_t (&k)[DIM],
                                         uint64_t& code) {
    if constexpr (DIM == 1) {
        code = static_cast<uint32_t>(k[0]);
        return true;
    } else if constexpr (DIM == 2) {
        const uint32_t u0 = static_cast<uint32_t>(k[0]) ^ 0x80000000u;
        const uint32_t u1 = static_cast<uint32_t>(k[1]) ^ 0x80000000u;
        code = static_cast<uint64_t>(u0) | (static_cast<uint64_t>(u1) << 32);
        return code < kTomb;
    } else if constexpr (DIM == 3) {
        const uint32_t u0 = static_cast<uint32_t>(k[0]) + (1u << 20);
        const uint32_t u1 = static_cast<uint32_t>(k[1]) + (1u << 20);
        const uint32_t u2 = static_cast<uint32_t>(k[2]) + (1u << 20);
        code = static_cast<uint64_t>(u0) | (static_cast<uint64_t>(u1) << 21) |
               (static_cast<uint64_t>(u2) << 42);
        return (u0 | u1 | u2) < (1u << 21);
    } else {
        const uint32_t u0 = static_cast<uint32_t>(k[0]) + 32768u;
        const uint32_t u1 = static_cast<uint32_t>(k[1]) + 32768u;
        const uint32_t u2 = static_cast<uint32_t>(k[2]) + 32768u;
        const uint32_t u3 = static_cast<uint32_t>(k[3]) + 32768u;
        code = static_cast<uint64_t>(u0) | (static_cast<uint64_t>(u1) << 16) |
               (static_cast<uint64_t>(u2) << 32) |
               (static_cast<uint64_t>(u3) << 48);
        return (u0 | u1 | u2 | u3) < 65536u && code < kTomb;
    }
}

template <int DIM>
__device__ __forceinline__ void unpack_key(uint64_t code, int32_t (&k)[DIM]) {
    if constexpr (DIM == 1) {
        k[0] = static_cast<int32_t>(static_cast<uint32_t>(code));
    } else if constexpr (DIM == 2) {
        k[0] = static_cast<int32_t>(static_cast<uint32_t>(code) ^ 0x80000000u);
        k[1] = static_cast<int32_t>(static_cast<uint32_t>(code >> 32) ^
                                    0x80000000u);
    } else if constexpr (DIM == 3) {
        k[0] = static_cast<int32_t>(code & 0x1FFFFFu) - (1 << 20);
        k[1] = static_cast<int32_t>((code >> 21) & 0x1FFFFFu) - (1 << 20);
        k[2] = static_cast<int32_t>((code >> 42) & 0x1FFFFFu) - (1 << 20);
    } else {
        k[0] = static_cast<int32_t>(code & 0xFFFFu) - 32768;
        k[1] = static_cast<int32_t>((code >> 16) & 0xFFFFu) - 32768;
        k[2] = static_cast<int32_t>((code >> 32) & 0xFFFFu) - 32768;
        k[3] = static_cast<int32_t>((code >> 48) & 0xFFFFu) - 32768;
    }
}

__device__ __forceinline__ uint64_t mix64(uint64_t h) {
    h ^= h >> 33;
    h *= 0xff51afd7ed558ccdull;
    h ^= h >> 33;
    h *= 0xc4ceb9fe1a85ec53ull;
    h ^= h >> 33;
    return h;
}

__device__ __forceinline__ uint32_t bucket_of(uint64_t code, uint32_t nb) {
    return __umulhi(static_cast<uint32_t>(mix64(code) >> 32), nb);
}

// The bucket after b in b's probe sequence: the next one of b's aligned range
// of kPartBuckets buckets, wrapping inside that range (a table of fewer
// buckets is one shorter range).  A sequence visits at most kPartBuckets buckets.
__device__ __forceinline__ uint32_t next_bucket(uint32_t b, uint32_t nb) {
    const uint32_t n = b + 1;
    return ((n & (kPartBuckets - 1)) == 0 || n == nb) ? (b & ~(kPartBuckets - 1)) : n;
}

template <int DIM>
__device__ __forceinline__ void load_key(const int32_t* __restrict__ keys,
                                         int64_t i, bool active,
                                         int32_t (&k)[DIM]) {
#pragma unroll
    for (int d = 0; d < DIM; ++d) k[d] = active ? keys[i * DIM + d] : 0;
}

// Value rows copied by a fused insert: row i of src[v] goes to row `index` of
// dst[v]; rows are row_dwords[v] 32-bit words long.
struct ValueArgs {
    int n;
    const uint32_t* src[kMaxFusedValues];
    uint32_t* dst[kMaxFusedValues];
    int32_t row_dwords[kMaxFusedValues];
};

// ---------------------------------------------------------------- host
struct DeviceGuard {
    int prev = -1;
    bool switched = false;
    hipError_t enter(int device) {
        hipError_t e = hipGetDevice(&prev);
        if (e != hipSuccess) return e;
        if (prev != device) {
            e = hipSetDevice(device);
            switched = (e == hipSuccess);
        }
        return e;
    }
    ~DeviceGuard() {
        if (switched) (void)hipSetDevice(prev);
    }
};

// The entry points that take tensors but no map (queries, convolution, surface
// extraction, depth integration) run on the device that holds their first
// tensor: the runtime is asked where the pointer lives and that device is made
// current for the call.  A pointer the runtime does not know leaves the
// current device as it is.
struct PointerGuard : DeviceGuard {
    hipError_t enter_for(const void* p) {
        if (p == nullptr) return hipSuccess;
        hipPointerAttribute_t attr;
        if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
            (void)hipGetLastError();
            return hipSuccess;
        }
        if (attr.type != hipMemoryTypeDevice) return hipSuccess;
        return enter(attr.device);
    }
};

// Inserts the keys selected by `sel[0 .. *nsel)` (both on the device) with the
// per-key atomic kernel.  `codes` false: `keys` are int32[.., key_dim] rows and
// sel holds row numbers; true: `keys` are packed 64-bit codes.  The value rows
// of va.src are addressed by the same selected row number.  Defined in
// ash_map.hip.
int insert_selected(ash_map* map, bool codes, const void* keys,
                    const int32_t* sel, const int32_t* nsel,
                    const ValueArgs& va, hipStream_t s);

// Erases the selected keys with the per-key kernel; arguments as for
// insert_selected.
int erase_selected(ash_map* map, bool codes, const void* keys, const int32_t* sel,
                   const int32_t* nsel, hipStream_t s);

int check_batch(const ash_map* map, const void* keys, int64_t n);
inline bool is_capturing(hipStream_t s) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    return hipStreamIsCapturing(s, &st) == hipSuccess && st != hipStreamCaptureStatusNone;
}

// Whether the heap array is known to be 0, 1, 2, ...
inline bool heap_in_order(const ash_map* map) { return !map->heap_dirty && !map->replayed; }

// What the host keeps of the counters no longer holds: `inserted` for a call
// that may have added entries (and ended without a look at the counters),
// false for one that took entries away.
// `s`: the stream the call runs on (captured: see ash_map::replayed).
void counters_changed(ash_map* map, bool inserted, hipStream_t s);
// The streaming insert (ash_bulk.hip); `early`, `early_event` as for
// ash_map_insert_bulk_early (both may be null).
int insert_bulk(ash_map* map, const int32_t* keys, int64_t n, int n_values,
                const void* const* src, void* const* dst, const int64_t* row_bytes,
                void* workspace, int64_t workspace_bytes, int32_t* early,
                hipEvent_t early_event, void* stream);
// Fills the bucket array if a clear() left that to the next user of the table.
int settle_table(ash_map* map, hipStream_t s);
// Before the first call that writes to the heap (an erase; a load brings a
// heap of its own): from here on items() reads the whole key log, so what a
// clear() left in it beyond the size is emptied now.
int give_up_heap_order(ash_map* map, hipStream_t s);

}  // namespace ash
