// Memory-system probes of bench.py (built into bench_probes.so by
// bench.py's build_probes(); not part of libash_hip.so or its C ABI).  The hash
// kernels are bound by how many random 128-byte lines per second the device
// can read or update, not by streaming bandwidth; these kernels measure those
// ceilings on the device at hand so that the benchmark can price the table
// kernels against them.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

namespace {

std::string g_error;

#define PROBE_FAIL(msg)   \
    do {                  \
        g_error = (msg);  \
        return 1;         \
    } while (0)

constexpr int kBlock = 256;

__device__ __forceinline__ uint64_t mix64(uint64_t h) {
    h ^= h >> 33;
    h *= 0xff51afd7ed558ccdull;
    h ^= h >> 33;
    h *= 0xc4ceb9fe1a85ec53ull;
    h ^= h >> 33;
    return h;
}

// Every group of 8 lanes reads 8 pseudo-random 128-byte lines, 16 bytes per
// lane, all 8 reads in flight at once: the access pattern of a table probe.
__global__ __launch_bounds__(kBlock) void probe_line_reads(
        const uint4* __restrict__ buf, uint32_t nlines, int64_t n,
        uint32_t* __restrict__ sink, uint64_t seed) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const int lane = threadIdx.x & 63;
    const int j = lane & 7;
    const int gbase = lane & ~7;
    const uint32_t line = __umulhi(
            static_cast<uint32_t>(mix64(static_cast<uint64_t>(t) + seed) >> 32),
            nlines);
    uint4 v[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        const uint32_t lr = __shfl(line, gbase | r);
        v[r] = buf[static_cast<size_t>(lr) * 8 + j];
    }
    uint32_t s = 0;
#pragma unroll
    for (int r = 0; r < 8; ++r) s += v[r].x ^ v[r].y ^ v[r].z ^ v[r].w;
    if (t < n) sink[t] = s;
}

// Every group of 4 lanes reads 4 pseudo-random aligned 64-byte halves of
// lines, 16 bytes per lane: what a probe of a table with 64-byte buckets would
// fetch (n counts the halves).
__global__ __launch_bounds__(kBlock) void probe_half_line_reads(
        const uint4* __restrict__ buf, uint32_t nlines, int64_t n,
        uint32_t* __restrict__ sink, uint64_t seed) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const int lane = threadIdx.x & 63;
    const int j = lane & 3;
    const int gbase = lane & ~3;
    const uint64_t h = mix64(static_cast<uint64_t>(t) + seed);
    const uint32_t half = 2u * __umulhi(static_cast<uint32_t>(h >> 32), nlines) +
                          (static_cast<uint32_t>(h) & 1u);
    uint4 v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t hr = __shfl(half, gbase | r);
        v[r] = buf[static_cast<size_t>(hr) * 4 + j];
    }
    uint32_t s = 0;
#pragma unroll
    for (int r = 0; r < 4; ++r) s += v[r].x ^ v[r].y ^ v[r].z ^ v[r].w;
    if (t < n) sink[t] = s;
}

// One thread per line: read one 64-bit word, compare-and-swap it, store one
// dword elsewhere in the line -- the three accesses an insert makes.
__global__ __launch_bounds__(kBlock) void probe_line_updates(
        unsigned long long* __restrict__ buf, uint32_t nlines, int64_t n,
        uint32_t* __restrict__ sink, uint64_t seed) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const uint64_t key = mix64(static_cast<uint64_t>(t) + seed);
    const uint32_t line = __umulhi(static_cast<uint32_t>(key >> 32), nlines);
    const int slot = static_cast<int>(key % 10);
    unsigned long long* p = buf + static_cast<size_t>(line) * 16 + slot;
    const unsigned long long seen = *p;
    const unsigned long long old = atomicCAS(p, seen, key | 1ull);
    reinterpret_cast<uint32_t*>(buf + static_cast<size_t>(line) * 16)[20 + slot] =
            static_cast<uint32_t>(t);
    if (t < n) sink[t] = static_cast<uint32_t>(old);
}

// Float adds without a result, the accumulation of a gradient: every group of
// GROUP neighbouring lanes adds to GROUP consecutive floats of one
// pseudo-random aligned piece of a 64-byte line (GROUP = 1: a lone float,
// GROUP = 16: a whole line).  Shows what the memory side charges for: the
// float, or the request one instruction sends to one line.
template <int GROUP>
__global__ __launch_bounds__(kBlock) void probe_float_adds(
        float* __restrict__ buf, uint32_t nlines, uint64_t seed) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const uint64_t h = mix64(static_cast<uint64_t>(t / GROUP) + seed);
    const uint32_t line = __umulhi(static_cast<uint32_t>(h >> 32), nlines);
    const uint32_t piece = (static_cast<uint32_t>(h) % (16u / GROUP)) * GROUP;
    // half-lines of 64 bytes: line numbers count 128-byte lines
    float* p = buf + static_cast<size_t>(line) * 32 + (static_cast<uint32_t>(h >> 8) & 1u) * 16 +
               piece + static_cast<uint32_t>(t % GROUP);
    __hip_atomic_fetch_add(p, 1.0f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace

extern "C" const char* bench_probe_last_error(void) { return g_error.c_str(); }

// `buf` is a 128-byte aligned device buffer of `buf_bytes` bytes treated as
// 128-byte lines; `n` (a multiple of 256) pseudo-random lines are touched and
// `sink` (uint32[n]) receives values that keep the accesses alive.  The caller
// times the call.
//   mode 0: every line is read in full by 8 lanes x 16 bytes (a table probe);
//   mode 1: per line one 64-bit read, one 64-bit compare-and-swap and one
//           32-bit store (the accesses of an insert); modifies `buf`;
//   mode 2: `n` pseudo-random aligned 64-byte halves of lines, each read by 4
//           lanes x 16 bytes (what a table of 64-byte buckets would fetch);
//   mode 3: `n` float adds (no result), every lane to a float of a line of
//           its own; modifies `buf`, `sink` is not written;
//   mode 4: `n` float adds, 16 neighbouring lanes to the 16 floats of one
//           64-byte half-line (n / 16 half-lines).
extern "C" int bench_probe_random_lines(int mode, void* buf, int64_t buf_bytes,
                                     int64_t n, uint32_t* sink, uint64_t seed,
                                     void* stream) {
    if (buf == nullptr || sink == nullptr) PROBE_FAIL("null buffer");
    if (buf_bytes < 128 || buf_bytes / 128 > 0xFFFFFFFFll) {
        PROBE_FAIL("buffer must hold between 1 and 2^32-1 lines of 128 bytes");
    }
    if (n <= 0 || n % kBlock != 0 || n > (int64_t{1} << 31)) {
        PROBE_FAIL("n must be a positive multiple of 256 below 2^31");
    }
    if (reinterpret_cast<uintptr_t>(buf) % 128 != 0) {
        PROBE_FAIL("buffer must be 128-byte aligned");
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint32_t nlines = static_cast<uint32_t>(buf_bytes / 128);
    const unsigned g = static_cast<unsigned>(n / kBlock);
    if (mode == 0) {
        probe_line_reads<<<g, kBlock, 0, s>>>(static_cast<const uint4*>(buf),
                                              nlines, n, sink, seed);
    } else if (mode == 1) {
        probe_line_updates<<<g, kBlock, 0, s>>>(
                static_cast<unsigned long long*>(buf), nlines, n, sink, seed);
    } else if (mode == 2) {
        probe_half_line_reads<<<g, kBlock, 0, s>>>(static_cast<const uint4*>(buf),
                                                   nlines, n, sink, seed);
    } else if (mode == 3) {
        probe_float_adds<1><<<g, kBlock, 0, s>>>(static_cast<float*>(buf), nlines, seed);
    } else if (mode == 4) {
        probe_float_adds<16><<<g, kBlock, 0, s>>>(static_cast<float*>(buf), nlines, seed);
    } else {
        PROBE_FAIL("unknown probe mode");
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) PROBE_FAIL(hipGetErrorString(e));
    return 0;
}
