/*
 * ash_oracle.c -- CPU restatement of torch-ash's hash map, trilinear query and
 * the grid functions around them.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker for the HIP library: it
 * is called from tests/, from __graft_entry__.smoke() and from the
 * `cpu_baseline` leg of bench.py, and from nowhere else.  The product never
 * links, loads or falls back to it.
 *
 * What it restates
 *   - the kernels and heap protocol of ash/src/hashmap_gpu.cuh (find :163-178,
 *     insert :211-232 and :249-283, erase :316-336, clear :354-358 with
 *     ash/src/hashmap_impl.h:26-33, items :360-405, load_states :407-450),
 *     executed as plain loops over the keys;
 *   - the container those kernels call, stdgpu::unordered_map.  stdgpu is a
 *     third-party submodule that is NOT vendored in the reference
 *     (.gitmodules:1-3, ext/stdgpu empty, version not pinned), so its published
 *     design is restated instead: `bucket_count` (a power of two) head slots
 *     followed by an excess region; a key hashes to head slot
 *     hash & (bucket_count-1); colliding keys are chained through per-slot
 *     offsets into slots popped from a stack of free excess positions; one
 *     lock per bucket serialises writers.  The hash is the reference's own
 *     MiniVecHash (ash/src/dispatch.h:110-123) and equality its MiniVecEq
 *     (:125-141).  Slot order is an stdgpu detail that no caller can observe
 *     except through the order of items(), which every caller sorts away.
 *   - the three query kernels of ash/src/grid.cu (:68-132, :177-255, :309-387)
 *     with their interpolation functors (:7-41), in the same operation order
 *     and in the same scalar type;
 *   - the callers either side of those paths: the ray marches of
 *     ash/src/sampler.cu, the sparse convolution (grid.cu:951-1006), the
 *     iso-surface point extraction (grid.cu:453-531) and marching cubes
 *     (grid.cu:606-946), each described at its function below.
 *
 * Marching cubes: the functions take the 256-row case table as an argument.
 * The Python face passes the reference's triangles (ash/src/mc_macros.h:32-288
 * in the reversed order of ash/src/grid.cu:818-841), re-expressed in the corner
 * and edge numbering used here and kept as a fixture under tests/golden/ by the
 * script that reads the reference's header as text.  The library's own table
 * comes from its generator and is compared with that fixture case by case.
 *
 * Where the reference has undefined behaviour (inserting more distinct keys
 * than `capacity` reads past the heap, ash/src/hashmap_gpu.cuh:226-227) the
 * restatement refuses the key and counts it in `dropped`.
 *
 * Parity pins: see tests/test_oracle_*.py (dictionary model, the invariants of
 * the reference's unittests, closed forms, torch.nn.functional.grid_sample,
 * float64 autograd of an independent formula, finite differences; hand-derived
 * marches, dense conv3d, spheres / tori / brute-force counts for the surface
 * functions).
 *
 * With OpenMP (-fopenmp) the loops over keys / queries run in parallel, which
 * is what bench.py times as the CPU baseline; with one thread the key loops
 * are strictly sequential and deterministic.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ASH_MAX_DIM 4

typedef struct ash_oracle_map {
    int dim;
    int64_t capacity;
    int64_t bucket_count; /* power of two */
    int64_t total_count;  /* bucket_count + excess_count */
    int32_t* keys;        /* total_count * dim */
    int32_t* values;      /* total_count */
    int64_t* next;        /* total_count: next slot of the chain, -1 = end */
    uint8_t* occupied;    /* total_count */
    int32_t* locks;       /* bucket_count */
    int64_t* excess;      /* stack of free excess positions */
    int64_t excess_top;   /* number of free positions on the stack */
    int64_t size;
    int64_t dropped;
    int32_t* heap;        /* caller-owned, capacity entries */
    int32_t heap_counter;
} ash_oracle_map;

/* ash/src/dispatch.h:110-123: FNV-1a style, elements sign-extended to 64 bit. */
static uint64_t key_hash(const int32_t* key, int dim) {
    uint64_t hash = UINT64_C(14695981039346656037);
    for (int i = 0; i < dim; ++i) {
        hash ^= (uint64_t)(int64_t)key[i];
        hash *= UINT64_C(1099511628211);
    }
    return hash;
}

/* ash/src/dispatch.h:125-141 */
static int key_equal(const int32_t* a, const int32_t* b, int dim) {
    int eq = 1;
    for (int i = 0; i < dim; ++i) eq = eq && (a[i] == b[i]);
    return eq;
}

static void reset_container(ash_oracle_map* m) {
    memset(m->occupied, 0, (size_t)m->total_count);
    for (int64_t i = 0; i < m->total_count; ++i) m->next[i] = -1;
    memset(m->locks, 0, (size_t)m->bucket_count * sizeof(int32_t));
    int64_t n_excess = m->total_count - m->bucket_count;
    for (int64_t i = 0; i < n_excess; ++i) {
        m->excess[i] = m->total_count - 1 - i; /* lowest position on top */
    }
    m->excess_top = n_excess;
    m->size = 0;
}

/* ash/src/hashmap_impl.h:26-33 */
static void reset_heap(ash_oracle_map* m) {
    m->heap_counter = 0;
    for (int64_t i = 0; i < m->capacity; ++i) m->heap[i] = (int32_t)i;
}

ash_oracle_map* ash_oracle_map_create(int dim, int64_t capacity, int32_t* heap) {
    if (dim < 1 || dim > ASH_MAX_DIM || capacity < 1 || heap == NULL) return NULL;
    ash_oracle_map* m = (ash_oracle_map*)calloc(1, sizeof(ash_oracle_map));
    if (!m) return NULL;
    m->dim = dim;
    m->capacity = capacity;
    int64_t b = 1;
    while (b < capacity) b <<= 1;
    m->bucket_count = b;
    /* every key may collide: keep room for `capacity` chained entries */
    m->total_count = b + capacity;
    m->keys = (int32_t*)malloc((size_t)m->total_count * dim * sizeof(int32_t));
    m->values = (int32_t*)malloc((size_t)m->total_count * sizeof(int32_t));
    m->next = (int64_t*)malloc((size_t)m->total_count * sizeof(int64_t));
    m->occupied = (uint8_t*)malloc((size_t)m->total_count);
    m->locks = (int32_t*)malloc((size_t)b * sizeof(int32_t));
    m->excess = (int64_t*)malloc((size_t)capacity * sizeof(int64_t));
    m->heap = heap;
    if (!m->keys || !m->values || !m->next || !m->occupied || !m->locks ||
        !m->excess) {
        free(m->keys); free(m->values); free(m->next); free(m->occupied);
        free(m->locks); free(m->excess); free(m);
        return NULL;
    }
    reset_container(m);
    reset_heap(m);
    m->dropped = 0;
    return m;
}

void ash_oracle_map_destroy(ash_oracle_map* m) {
    if (!m) return;
    free(m->keys); free(m->values); free(m->next); free(m->occupied);
    free(m->locks); free(m->excess); free(m);
}

static void lock_bucket(ash_oracle_map* m, int64_t b) {
    int32_t expected = 0;
    while (!__atomic_compare_exchange_n(&m->locks[b], &expected, 1, 0,
                                        __ATOMIC_ACQUIRE, __ATOMIC_RELAXED)) {
        expected = 0;
    }
}

static void unlock_bucket(ash_oracle_map* m, int64_t b) {
    __atomic_store_n(&m->locks[b], 0, __ATOMIC_RELEASE);
}

/* Chain walk; returns the slot holding `key` or -1.  *last receives the final
 * slot of the chain (or -1 when the head slot itself is free). */
static int64_t chain_find(const ash_oracle_map* m, int64_t bucket,
                          const int32_t* key, int64_t* last) {
    int64_t slot = bucket;
    int64_t tail = -1;
    /* the head slot may be free while its chain continues (after an erase) */
    while (slot >= 0) {
        if (m->occupied[slot] &&
            key_equal(m->keys + slot * m->dim, key, m->dim)) {
            if (last) *last = tail;
            return slot;
        }
        tail = slot;
        slot = m->next[slot];
    }
    if (last) *last = tail;
    return -1;
}

/* emplace: returns the slot and whether it was newly created; -1 when the
 * key is new but cannot be stored.  With `from_heap` the value of a new entry
 * is the next free index, heap[heap_counter++]: the reference first emplaces a
 * dummy 0 and overwrites it with the popped index right after
 * (ash/src/hashmap_gpu.cuh:222-231); popping before the entry becomes visible
 * gives the same map and lets an exhausted heap refuse the key cleanly. */
static int64_t emplace(ash_oracle_map* m, const int32_t* key, int32_t value,
                       int from_heap, int* inserted) {
    int64_t bucket = (int64_t)(key_hash(key, m->dim) &
                               (uint64_t)(m->bucket_count - 1));
    *inserted = 0;
    lock_bucket(m, bucket);
    int64_t tail = -1;
    int64_t slot = chain_find(m, bucket, key, &tail);
    if (slot < 0) {
        if (from_heap) {
            int32_t top =
                    __atomic_fetch_add(&m->heap_counter, 1, __ATOMIC_RELAXED);
            if (top >= m->capacity) {
                __atomic_fetch_sub(&m->heap_counter, 1, __ATOMIC_RELAXED);
                unlock_bucket(m, bucket);
                return -1;
            }
            value = m->heap[top];
        }
        if (!m->occupied[bucket]) {
            slot = bucket;
        } else {
            int64_t top;
#ifdef _OPENMP
#pragma omp atomic capture
#endif
            top = --m->excess_top;
            /* cannot run dry: there are `capacity` excess positions and at
             * most `capacity` live entries */
            slot = m->excess[top];
            m->next[slot] = -1;
            m->next[tail] = slot; /* append to the chain */
        }
        memcpy(m->keys + slot * m->dim, key, (size_t)m->dim * sizeof(int32_t));
        m->values[slot] = value;
        m->occupied[slot] = 1;
#ifdef _OPENMP
#pragma omp atomic
#endif
        m->size++;
        *inserted = 1;
    }
    unlock_bucket(m, bucket);
    return slot;
}

static int64_t lookup(const ash_oracle_map* m, const int32_t* key) {
    int64_t bucket = (int64_t)(key_hash(key, m->dim) &
                               (uint64_t)(m->bucket_count - 1));
    return chain_find(m, bucket, key, NULL);
}

/* erase(key): 1 when this call removed the entry. */
static int erase_one(ash_oracle_map* m, const int32_t* key, int32_t* value) {
    int64_t bucket = (int64_t)(key_hash(key, m->dim) &
                               (uint64_t)(m->bucket_count - 1));
    lock_bucket(m, bucket);
    int64_t prev = -1;
    int64_t slot = chain_find(m, bucket, key, &prev);
    int removed = 0;
    if (slot >= 0) {
        *value = m->values[slot];
        m->occupied[slot] = 0;
        if (slot != bucket) {
            /* unlink an excess slot and give it back */
            m->next[prev] = m->next[slot];
            m->next[slot] = -1;
            int64_t top;
#ifdef _OPENMP
#pragma omp atomic capture
#endif
            top = m->excess_top++;
            m->excess[top] = slot;
        }
#ifdef _OPENMP
#pragma omp atomic
#endif
        m->size--;
        removed = 1;
    }
    unlock_bucket(m, bucket);
    return removed;
}

/* ash/src/hashmap_gpu.cuh:163-178 */
void ash_oracle_map_find(const ash_oracle_map* m, const int32_t* keys, int64_t n,
                         int64_t* indices, uint8_t* masks) {
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (int64_t tid = 0; tid < n; ++tid) {
        int64_t slot = lookup(m, keys + tid * m->dim);
        int flag = slot >= 0;
        masks[tid] = (uint8_t)flag;
        indices[tid] = flag ? (int64_t)m->values[slot] : 0;
    }
}

/* One thread of insert_kernel (ash/src/hashmap_gpu.cuh:211-232, :249-283).
 * Returns the index given to the key, -1 when it was already present or
 * refused because the heap is exhausted (undefined in the reference). */
static int32_t insert_one(ash_oracle_map* m, const int32_t* key) {
    int inserted = 0;
    int64_t slot = emplace(m, key, 0, 1, &inserted);
    if (slot < 0) {
#ifdef _OPENMP
#pragma omp atomic
#endif
        m->dropped++;
        return -1;
    }
    return inserted ? m->values[slot] : -1;
}

void ash_oracle_map_insert_keys(ash_oracle_map* m, const int32_t* keys,
                                int64_t n) {
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (int64_t tid = 0; tid < n; ++tid) insert_one(m, keys + tid * m->dim);
}

/* ash/src/hashmap_gpu.cuh:249-313: rows are moved as raw bytes; the blob width
 * rule (:79-114) only picks the copy granularity and cannot change the result. */
void ash_oracle_map_insert(ash_oracle_map* m, const int32_t* keys, int64_t n,
                           int n_values, const void* const* src,
                           void* const* dst, const int64_t* row_bytes) {
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (int64_t tid = 0; tid < n; ++tid) {
        int32_t idx = insert_one(m, keys + tid * m->dim);
        if (idx < 0) continue;
        for (int j = 0; j < n_values; ++j) {
            memcpy((char*)dst[j] + (int64_t)idx * row_bytes[j],
                   (const char*)src[j] + tid * row_bytes[j],
                   (size_t)row_bytes[j]);
        }
    }
}

/* ash/src/hashmap_gpu.cuh:316-336 */
void ash_oracle_map_erase(ash_oracle_map* m, const int32_t* keys, int64_t n) {
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (int64_t tid = 0; tid < n; ++tid) {
        int32_t value = 0;
        if (erase_one(m, keys + tid * m->dim, &value)) {
            int32_t top = __atomic_fetch_sub(&m->heap_counter, 1, __ATOMIC_RELAXED);
            m->heap[top - 1] = value;
        }
    }
}

/* ash/src/hashmap_gpu.cuh:354-358 */
void ash_oracle_map_clear(ash_oracle_map* m) {
    reset_container(m);
    reset_heap(m);
    m->dropped = 0;
}

int64_t ash_oracle_map_size(const ash_oracle_map* m) { return m->size; }
int64_t ash_oracle_map_dropped(const ash_oracle_map* m) { return m->dropped; }

/* ash/src/hashmap_gpu.cuh:360-405: occupied slots in slot order. */
int64_t ash_oracle_map_items(const ash_oracle_map* m, int32_t* keys_out,
                             int64_t* indices_out) {
    int64_t n = 0;
    for (int64_t s = 0; s < m->total_count; ++s) {
        if (!m->occupied[s]) continue;
        memcpy(keys_out + n * m->dim, m->keys + s * m->dim,
               (size_t)m->dim * sizeof(int32_t));
        indices_out[n] = (int64_t)m->values[s];
        ++n;
    }
    return n;
}

/* ash/src/hashmap_gpu.cuh:407-450.  Returns the number of pairs that could not
 * be stored because their key was already present (the reference prints an
 * error for those).  Unlike the reference the container is emptied first. */
int64_t ash_oracle_map_load(ash_oracle_map* m, const int32_t* keys,
                            const int64_t* indices, int64_t n,
                            const int32_t* heap_src) {
    reset_container(m);
    m->dropped = 0;
    m->heap_counter = (int32_t)n;
    if (heap_src != NULL && heap_src != m->heap) {
        memcpy(m->heap, heap_src, (size_t)m->capacity * sizeof(int32_t));
    }
    int64_t failed = 0;
    for (int64_t tid = 0; tid < n; ++tid) {
        int inserted = 0;
        int64_t slot = emplace(m, keys + tid * m->dim, (int32_t)indices[tid], 0,
                               &inserted);
        if (slot < 0 || !inserted) ++failed;
    }
    return failed;
}

/* ------------------------------------------------------------------------ */
/* Trilinear query (ash/src/grid.cu).  Instantiated for float and double.    */

#define ASH_INTERP_LINEAR 0
#define ASH_INTERP_SMOOTH_STEP 1

#define DEFINE_QUERY(T, SUFFIX)                                                \
    /* ash/src/grid.cu:7-41 */                                                 \
    static T interp_##SUFFIX(T x, int kind) {                                  \
        return kind == ASH_INTERP_SMOOTH_STEP ? x * x * (3 - 2 * x) : x;       \
    }                                                                          \
    static T diff_interp_##SUFFIX(T x, int kind) {                             \
        return kind == ASH_INTERP_SMOOTH_STEP ? 6 * x * (1 - x) : (T)1;        \
    }                                                                          \
                                                                               \
    /* ash/src/grid.cu:68-132; output is zero-initialised as at :153 */        \
    void ash_oracle_query_forward_##SUFFIX(                                    \
            const T* embeddings, const float* offsets,                         \
            const int64_t* grid_indices, const int64_t* cell_indices,          \
            const uint8_t* masks, const int64_t* lut_grid_nb2grid_idx,         \
            const int64_t* lut_cell_nb2cell_idx,                               \
            const int64_t* lut_cell_nb2grid_nb, T* output, int64_t len,        \
            int64_t cells_per_grid, int64_t embedding_dims, int kind) {        \
        memset(output, 0, (size_t)(len * embedding_dims) * sizeof(T));         \
        _Pragma("omp parallel for schedule(static)")                           \
        for (int64_t i = 0; i < len; ++i) {                                    \
            if (!masks[i]) continue;                                           \
            int64_t grid_idx = grid_indices[i];                                \
            int64_t cell_idx = cell_indices[i];                                \
            const float* offset = offsets + i * 3;                             \
            const int64_t* nb_g2g = lut_grid_nb2grid_idx + grid_idx * 8;       \
            const int64_t* nb_c2c = lut_cell_nb2cell_idx + cell_idx * 8;       \
            const int64_t* nb_c2g = lut_cell_nb2grid_nb + cell_idx * 8;        \
            T local_sum[16];                                                   \
            for (int k = 0; k < 16; ++k) local_sum[k] = 0;                     \
            int complete = 1;                                                  \
            for (int cell_nb = 0; cell_nb < 8; ++cell_nb) {                    \
                int64_t grid_nb = nb_c2g[cell_nb];                             \
                int64_t grid_nb_idx = nb_g2g[grid_nb];                         \
                if (grid_nb_idx == -1) {                                       \
                    complete = 0;                                              \
                    break;                                                     \
                }                                                              \
                T weight = 1.0;                                                \
                for (int d = 0; d < 3; ++d) {                                  \
                    int dim_code = (cell_nb >> d) & 1;                         \
                    T x = dim_code ? (offset[d]) : (1 - offset[d]);            \
                    weight *= interp_##SUFFIX(x, kind);                        \
                }                                                              \
                int64_t cell_nb_idx = nb_c2c[cell_nb];                         \
                int64_t base_idx = (grid_nb_idx * cells_per_grid +             \
                                    cell_nb_idx) * embedding_dims;             \
                for (int64_t k = 0; k < embedding_dims; ++k) {                 \
                    local_sum[k] += weight * embeddings[base_idx + k];         \
                }                                                              \
            }                                                                  \
            if (!complete) continue;                                           \
            for (int64_t k = 0; k < embedding_dims; ++k) {                     \
                output[i * embedding_dims + k] = local_sum[k];                 \
            }                                                                  \
        }                                                                      \
    }                                                                          \
                                                                               \
    /* ash/src/grid.cu:177-255; outputs zero-initialised as at :273-274 */     \
    void ash_oracle_query_backward_forward_##SUFFIX(                           \
            const T* z, const T* embeddings, const float* offsets,             \
            const int64_t* grid_indices, const int64_t* cell_indices,          \
            const uint8_t* masks, const int64_t* lut_grid_nb2grid_idx,         \
            const int64_t* lut_cell_nb2cell_idx,                               \
            const int64_t* lut_cell_nb2grid_nb, T* grad_embeddings,            \
            T* grad_offsets, int64_t len, int64_t num_embeddings,              \
            int64_t cells_per_grid, int64_t embedding_dims, int kind) {        \
        memset(grad_embeddings, 0,                                             \
               (size_t)(num_embeddings * cells_per_grid * embedding_dims) *    \
                       sizeof(T));                                             \
        memset(grad_offsets, 0, (size_t)(len * 3) * sizeof(T));                \
        _Pragma("omp parallel for schedule(static)")                           \
        for (int64_t i = 0; i < len; ++i) {                                    \
            if (!masks[i]) continue;                                           \
            int64_t grid_idx = grid_indices[i];                                \
            int64_t cell_idx = cell_indices[i];                                \
            const float* offset = offsets + i * 3;                             \
            const int64_t* nb_g2g = lut_grid_nb2grid_idx + grid_idx * 8;       \
            const int64_t* nb_c2c = lut_cell_nb2cell_idx + cell_idx * 8;       \
            const int64_t* nb_c2g = lut_cell_nb2grid_nb + cell_idx * 8;        \
            int complete = 1;                                                  \
            for (int cell_nb = 0; cell_nb < 8; ++cell_nb) {                    \
                if (nb_g2g[nb_c2g[cell_nb]] == -1) complete = 0;               \
            }                                                                  \
            if (!complete) continue;                                           \
            for (int cell_nb = 0; cell_nb < 8; ++cell_nb) {                    \
                int64_t grid_nb_idx = nb_g2g[nb_c2g[cell_nb]];                 \
                T weight = 1.0;                                                \
                T weight_grad[3] = {1, 1, 1};                                  \
                for (int d = 0; d < 3; ++d) {                                  \
                    int dim_code = (cell_nb >> d) & 1;                         \
                    T x = dim_code ? (offset[d]) : (1 - offset[d]);            \
                    T w = interp_##SUFFIX(x, kind);                            \
                    T dw = diff_interp_##SUFFIX(x, kind) *                     \
                           (dim_code ? 1 : -1);                                \
                    weight *= w;                                               \
                    weight_grad[0] *= (d == 0) ? dw : w;                       \
                    weight_grad[1] *= (d == 1) ? dw : w;                       \
                    weight_grad[2] *= (d == 2) ? dw : w;                       \
                }                                                              \
                int64_t cell_nb_idx = nb_c2c[cell_nb];                         \
                int64_t base_idx = (grid_nb_idx * cells_per_grid +             \
                                    cell_nb_idx) * embedding_dims;             \
                T dot = 0.0;                                                   \
                for (int64_t k = 0; k < embedding_dims; ++k) {                 \
                    T z_k = z[i * embedding_dims + k];                         \
                    T contribution = weight * z_k;                             \
                    _Pragma("omp atomic")                                      \
                    grad_embeddings[base_idx + k] += contribution;             \
                    dot += embeddings[base_idx + k] * z_k;                     \
                }                                                              \
                for (int d = 0; d < 3; ++d) {                                  \
                    grad_offsets[i * 3 + d] += dot * weight_grad[d];           \
                }                                                              \
            }                                                                  \
        }                                                                      \
    }                                                                          \
                                                                               \
    /* ash/src/grid.cu:309-387; grad_z and grad_embeddings zero-initialised  */\
    /* as at :413-414; the offsets gradient stays zero (:417-418) and the    */\
    /* incoming grad_grad_embeddings is not an operand (:426).               */\
    void ash_oracle_query_backward_backward_##SUFFIX(                          \
            const T* grad_grad_offset, const T* z, const T* embeddings,        \
            const float* offsets, const int64_t* grid_indices,                 \
            const int64_t* cell_indices, const uint8_t* masks,                 \
            const int64_t* lut_grid_nb2grid_idx,                               \
            const int64_t* lut_cell_nb2cell_idx,                               \
            const int64_t* lut_cell_nb2grid_nb, T* grad_z,                     \
            T* grad_embeddings, int64_t len, int64_t num_embeddings,           \
            int64_t cells_per_grid, int64_t embedding_dims, int kind) {        \
        memset(grad_embeddings, 0,                                             \
               (size_t)(num_embeddings * cells_per_grid * embedding_dims) *    \
                       sizeof(T));                                             \
        memset(grad_z, 0, (size_t)(len * embedding_dims) * sizeof(T));         \
        _Pragma("omp parallel for schedule(static)")                           \
        for (int64_t i = 0; i < len; ++i) {                                    \
            if (!masks[i]) continue;                                           \
            int64_t grid_idx = grid_indices[i];                                \
            int64_t cell_idx = cell_indices[i];                                \
            const float* offset = offsets + i * 3;                             \
            const int64_t* nb_g2g = lut_grid_nb2grid_idx + grid_idx * 8;       \
            const int64_t* nb_c2c = lut_cell_nb2cell_idx + cell_idx * 8;       \
            const int64_t* nb_c2g = lut_cell_nb2grid_nb + cell_idx * 8;        \
            int complete = 1;                                                  \
            for (int cell_nb = 0; cell_nb < 8; ++cell_nb) {                    \
                if (nb_g2g[nb_c2g[cell_nb]] == -1) complete = 0;               \
            }                                                                  \
            if (!complete) continue;                                           \
            for (int cell_nb = 0; cell_nb < 8; ++cell_nb) {                    \
                int64_t grid_nb_idx = nb_g2g[nb_c2g[cell_nb]];                 \
                T weight_grad[3] = {1, 1, 1};                                  \
                for (int d = 0; d < 3; ++d) {                                  \
                    int dim_code = (cell_nb >> d) & 1;                         \
                    T x = dim_code ? (offset[d]) : (1 - offset[d]);            \
                    T w = interp_##SUFFIX(x, kind);                            \
                    T dw = diff_interp_##SUFFIX(x, kind) *                     \
                           (dim_code ? 1 : -1);                                \
                    weight_grad[0] *= (d == 0) ? dw : w;                       \
                    weight_grad[1] *= (d == 1) ? dw : w;                       \
                    weight_grad[2] *= (d == 2) ? dw : w;                       \
                }                                                              \
                int64_t cell_nb_idx = nb_c2c[cell_nb];                         \
                int64_t base_lhs = (grid_nb_idx * cells_per_grid +             \
                                    cell_nb_idx) * embedding_dims;             \
                int64_t base_rhs = i * embedding_dims;                         \
                T dot = 0;                                                     \
                for (int d = 0; d < 3; ++d) {                                  \
                    dot += weight_grad[d] * grad_grad_offset[i * 3 + d];       \
                }                                                              \
                for (int64_t k = 0; k < embedding_dims; ++k) {                 \
                    T contribution = dot * z[base_rhs + k];                    \
                    _Pragma("omp atomic")                                      \
                    grad_embeddings[base_lhs + k] += contribution;             \
                    grad_z[base_rhs + k] += dot * embeddings[base_lhs + k];    \
                }                                                              \
            }                                                                  \
        }                                                                      \
    }

DEFINE_QUERY(float, f32)
DEFINE_QUERY(double, f64)

/* Magnitudes behind the three query functions, for error bounds in the tests:
 * for every output element the sum of the ABSOLUTE values of the terms that
 * the kernels above add up to form it, in double.  A sum of n fp32 terms
 * evaluated in any order differs from the exact sum by at most about
 * n * 2^-24 * (sum of |terms|), so these are what a tolerance for sums that two
 * implementations accumulate in different orders has to scale with.  Same
 * addressing, early-outs and weights as the kernels (ash/src/grid.cu:68-132,
 * :177-255, :309-387); not a restatement of anything in the reference.
 *   sum_forward[i,k]      = sum_c w_c |emb_c[k]|
 *   sum_bf_emb[row,k]     = sum_i w_c |z[i,k]|              (row = corner c of query i)
 *   sum_bf_off[i,d]       = sum_c |dw_c/do_d| sum_k |emb_c[k] z[i,k]|
 *   sum_bb_z[i,k]         = sum_c (sum_d |dw_c/do_d u[i,d]|) |emb_c[k]|
 *   sum_bb_emb[row,k]     = sum_i (sum_d |dw_c/do_d u[i,d]|) |z[i,k]|
 * Any output may be NULL; z / u may be NULL when no output needs them. */
void ash_oracle_query_term_sums(
        const double* u, const double* z, const double* embeddings,
        const float* offsets, const int64_t* grid_indices,
        const int64_t* cell_indices, const uint8_t* masks,
        const int64_t* lut_grid_nb2grid_idx, const int64_t* lut_cell_nb2cell_idx,
        const int64_t* lut_cell_nb2grid_nb, double* sum_forward, double* sum_bf_emb,
        double* sum_bf_off, double* sum_bb_z, double* sum_bb_emb, int64_t len,
        int64_t num_embeddings, int64_t cells_per_grid, int64_t embedding_dims,
        int kind) {
    const size_t dense = (size_t)(num_embeddings * cells_per_grid * embedding_dims);
    if (sum_forward) memset(sum_forward, 0, (size_t)(len * embedding_dims) * sizeof(double));
    if (sum_bf_emb) memset(sum_bf_emb, 0, dense * sizeof(double));
    if (sum_bf_off) memset(sum_bf_off, 0, (size_t)(len * 3) * sizeof(double));
    if (sum_bb_z) memset(sum_bb_z, 0, (size_t)(len * embedding_dims) * sizeof(double));
    if (sum_bb_emb) memset(sum_bb_emb, 0, dense * sizeof(double));
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < len; ++i) {
        if (!masks[i]) continue;
        const float* offset = offsets + i * 3;
        const int64_t* nb_g2g = lut_grid_nb2grid_idx + grid_indices[i] * 8;
        const int64_t* nb_c2c = lut_cell_nb2cell_idx + cell_indices[i] * 8;
        const int64_t* nb_c2g = lut_cell_nb2grid_nb + cell_indices[i] * 8;
        int complete = 1;
        for (int c = 0; c < 8; ++c) {
            if (nb_g2g[nb_c2g[c]] == -1) complete = 0;
        }
        if (!complete) continue;
        for (int c = 0; c < 8; ++c) {
            double w = 1.0, wg[3] = {1, 1, 1};
            for (int d = 0; d < 3; ++d) {
                double x = ((c >> d) & 1) ? (double)offset[d] : (double)(1 - offset[d]);
                double f = interp_f64(x, kind);
                double df = fabs(diff_interp_f64(x, kind));
                w *= f;
                for (int e = 0; e < 3; ++e) wg[e] *= (e == d) ? df : f;
            }
            w = fabs(w);
            double du = 0;
            if (u) {
                for (int d = 0; d < 3; ++d) du += fabs(wg[d] * u[i * 3 + d]);
            }
            const int64_t base = (nb_g2g[nb_c2g[c]] * cells_per_grid + nb_c2c[c]) * embedding_dims;
            double dot = 0;
            for (int64_t k = 0; k < embedding_dims; ++k) {
                const double e_k = fabs(embeddings[base + k]);
                const double z_k = z ? fabs(z[i * embedding_dims + k]) : 0.0;
                if (sum_forward) sum_forward[i * embedding_dims + k] += w * e_k;
                if (sum_bf_emb) {
#pragma omp atomic
                    sum_bf_emb[base + k] += w * z_k;
                }
                dot += e_k * z_k;
                if (sum_bb_z) sum_bb_z[i * embedding_dims + k] += du * e_k;
                if (sum_bb_emb) {
#pragma omp atomic
                    sum_bb_emb[base + k] += du * z_k;
                }
            }
            if (sum_bf_off) {
                for (int d = 0; d < 3; ++d) sum_bf_off[i * 3 + d] += wg[d] * dot;
            }
        }
    }
}

/* ------------------------------------------------------- iso-surface points
 * ash/src/grid.cu:453-531, cells in launch order.  Returns the number of
 * points; positions (may be NULL) receives them in that order. */
#define ASH_ORACLE_ISOSURFACE(NAME, T)                                        \
    int64_t NAME(const T* sdfs, const T* weights, const int64_t* grid_indices, \
                 const int32_t* grid_coords, const int64_t* lut_g,            \
                 const int32_t* cell_coords, const int64_t* lut_c2c,          \
                 const int64_t* lut_c2g, int64_t n_grids, int64_t M, int g,   \
                 float iso, float weight_thr, float* positions) {             \
        int64_t count = 0;                                                    \
        for (int64_t i = 0; i < n_grids * M; ++i) {                           \
            const int64_t gi = grid_indices[i / M];                           \
            const int64_t c = i % M;                                          \
            if (weights[gi * M + c] < weight_thr) continue;                   \
            const T self = sdfs[gi * M + c] - iso;                            \
            for (int d = 0; d < 3; ++d) {                                     \
                const int nb = 1 << d;                                        \
                const int64_t ng = lut_g[gi * 8 + lut_c2g[c * 8 + nb]];       \
                if (ng == -1) break;                                          \
                const int64_t nc = lut_c2c[c * 8 + nb];                       \
                const T other = sdfs[ng * M + nc] - iso;                      \
                if (self * other < 0 && weights[ng * M + nc] >= weight_thr) { \
                    if (positions) {                                          \
                        const float ratio = (float)(self / (self - other));   \
                        for (int a = 0; a < 3; ++a) {                         \
                            positions[count * 3 + a] =                        \
                                    (float)(grid_coords[gi * 3 + a] * g +     \
                                            cell_coords[c * 3 + a]) +         \
                                    (a == d ? ratio : 0.f);                   \
                        }                                                     \
                    }                                                         \
                    ++count;                                                  \
                }                                                             \
            }                                                                 \
        }                                                                     \
        return count;                                                         \
    }
ASH_ORACLE_ISOSURFACE(ash_oracle_isosurface_f32, float)
ASH_ORACLE_ISOSURFACE(ash_oracle_isosurface_f64, double)

/* ---------------------------------------------------------- marching cubes
 * ash/src/grid.cu:606-946 in launch order: case per cell and placeholders on
 * the owning cells of crossed edges (:606-703), vertex ids and positions
 * (:705-774), triangles (:776-842).  Corner c of a cell is entry c of the
 * 8-entry neighbour tables and bit c of the case (the reference reaches the
 * same cells through its own corner numbering, grid.cu:646-666); edge
 * e = 4 * axis + j starts at the corner made by inserting a zero bit at
 * position `axis` into j.  `table` holds, per case, up to five triangles as
 * edge triples in output order, -1 padded to 16.  `case_ws` int32[B * M] and
 * `edge_ws` int32[B * M * 3] are work arrays.  positions / triangles may be
 * NULL to count only; counts[0] = vertices, counts[1] = triangles. */
static int mc_low_corner(int e) {
    const int axis = e >> 2, j = e & 3;
    return (j & ((1 << axis) - 1)) | ((j >> axis) << (axis + 1));
}

#define ASH_ORACLE_MARCHING_CUBES(NAME, T)                                     \
    void NAME(const T* sdfs, const T* weights, const int64_t* grid_indices,    \
              const int32_t* grid_coords, const int64_t* lut_g,                \
              const int32_t* cell_coords, const int64_t* lut_c2c,              \
              const int64_t* lut_c2g, int64_t n_grids, int64_t B, int64_t M,   \
              int g, float iso, float weight_thr, const int8_t* table,         \
              int32_t* case_ws, int32_t* edge_ws, int64_t* counts,             \
              float* positions, int32_t* triangles) {                          \
        memset(case_ws, 0, sizeof(int32_t) * (size_t)(B * M));                 \
        memset(edge_ws, 0, sizeof(int32_t) * (size_t)(B * M * 3));             \
        for (int64_t i = 0; i < n_grids * M; ++i) {                            \
            const int64_t gi = grid_indices[i / M];                            \
            const int64_t c = i % M;                                           \
            if (weights[gi * M + c] < weight_thr) continue;                    \
            int code = 0, valid = 1;                                           \
            int64_t at[8];                                                     \
            for (int k = 0; k < 8 && valid; ++k) {                             \
                const int64_t ng = lut_g[gi * 8 + lut_c2g[c * 8 + k]];         \
                if (ng == -1) { valid = 0; break; }                            \
                at[k] = ng * M + lut_c2c[c * 8 + k];                           \
                if (weights[at[k]] < weight_thr) { valid = 0; break; }         \
                code |= ((sdfs[at[k]] - iso) < 0) << k;                        \
            }                                                                  \
            if (!valid || code == 0 || code == 255) continue;                  \
            case_ws[gi * M + c] = code;                                        \
            for (int e = 0; e < 12; ++e) {                                     \
                const int lo = mc_low_corner(e), hi = lo | (1 << (e >> 2));    \
                if (((code >> lo) ^ (code >> hi)) & 1) {                       \
                    edge_ws[at[lo] * 3 + (e >> 2)] = -1;                       \
                }                                                              \
            }                                                                  \
        }                                                                      \
        int64_t nv = 0, nt = 0;                                                \
        for (int64_t i = 0; i < n_grids * M; ++i) {                            \
            const int64_t gi = grid_indices[i / M];                            \
            const int64_t c = i % M;                                           \
            const T self = sdfs[gi * M + c] - iso;                             \
            for (int d = 0; d < 3; ++d) {                                      \
                if (edge_ws[(gi * M + c) * 3 + d] != -1) continue;             \
                const int64_t ng = lut_g[gi * 8 + lut_c2g[c * 8 + (1 << d)]];  \
                const int64_t nc = lut_c2c[c * 8 + (1 << d)];                  \
                const T other = sdfs[ng * M + nc] - iso;                       \
                if (positions) {                                               \
                    const float ratio = (float)(self / (self - other));        \
                    for (int a = 0; a < 3; ++a) {                              \
                        positions[nv * 3 + a] =                                \
                                (float)(grid_coords[gi * 3 + a] * g +          \
                                        cell_coords[c * 3 + a]) +              \
                                (a == d ? ratio : 0.f);                        \
                    }                                                          \
                }                                                              \
                edge_ws[(gi * M + c) * 3 + d] = (int32_t)nv++;                 \
            }                                                                  \
        }                                                                      \
        for (int64_t i = 0; i < n_grids * M; ++i) {                            \
            const int64_t gi = grid_indices[i / M];                            \
            const int64_t c = i % M;                                           \
            const int code = case_ws[gi * M + c];                              \
            if (code == 0) continue;                                           \
            for (int t = 0; t < 15 && table[code * 16 + t] != -1; t += 3) {    \
                for (int v = 0; v < 3 && triangles; ++v) {                     \
                    const int e = table[code * 16 + t + v];                    \
                    const int lo = mc_low_corner(e);                           \
                    const int64_t ng = lut_g[gi * 8 + lut_c2g[c * 8 + lo]];    \
                    const int64_t nc = lut_c2c[c * 8 + lo];                    \
                    triangles[nt * 3 + v] = edge_ws[(ng * M + nc) * 3 + (e >> 2)]; \
                }                                                              \
                ++nt;                                                          \
            }                                                                  \
        }                                                                      \
        counts[0] = nv;                                                        \
        counts[1] = nt;                                                        \
    }
ASH_ORACLE_MARCHING_CUBES(ash_oracle_marching_cubes_f32, float)
ASH_ORACLE_MARCHING_CUBES(ash_oracle_marching_cubes_f64, double)

/* ----------------------------------------------------------- convolution
 * ash/src/grid.cu:951-1006: taps accumulated in table order, one fused
 * multiply-add per tap and channel (nvcc's contraction of `sum += in * w`). */
#define ASH_ORACLE_CONVOLUTION(NAME, T, FMA)                                   \
    void NAME(const T* in, const T* w, const uint8_t* masks,                  \
              const int64_t* grid_indices, const int64_t* cell_indices,       \
              const int64_t* lut_g, const int64_t* lut_c2c,                   \
              const int64_t* lut_c2g, T* out, int64_t n_grids, int64_t B,     \
              int64_t M, int64_t E, int64_t K, int64_t GN) {                  \
        memset(out, 0, (size_t)(B * M * E) * sizeof(T));                      \
        _Pragma("omp parallel for schedule(static)")                          \
        for (int64_t i = 0; i < n_grids * M; ++i) {                           \
            if (!masks[i]) continue;                                          \
            const int64_t g = grid_indices[i / M];                            \
            const int64_t c = cell_indices[i % M];                            \
            T* o = out + (g * M + c) * E;                                     \
            for (int64_t k = 0; k < K; ++k) {                                 \
                const int64_t gi = lut_g[g * GN + lut_c2g[c * K + k]];        \
                if (gi < 0) continue;                                         \
                const T* row = in + (gi * M + lut_c2c[c * K + k]) * E;        \
                for (int64_t e = 0; e < E; ++e) {                             \
                    o[e] = FMA(row[e], w[k * E + e], o[e]);                   \
                }                                                             \
            }                                                                 \
        }                                                                     \
    }
ASH_ORACLE_CONVOLUTION(ash_oracle_convolution_forward_f32, float, fmaf)
ASH_ORACLE_CONVOLUTION(ash_oracle_convolution_forward_f64, double, fma)

/* ------------------------------------------------------------------ rays
 * ash/src/sampler.cu:7-67 and :122-214, one loop iteration per kernel thread.
 * Positions are `origin + t * direction`; nvcc contracts that expression into
 * a fused multiply-add, restated with fmaf() so that every implementation
 * checked against this file rounds alike.  Everything is in cell units; a
 * block is `grid2cell` cells wide. */
void ash_oracle_ray_find_near_far(const ash_oracle_map* m, const float* origins,
                                  const float* directions, const float* bbox_min,
                                  const float* bbox_max, int64_t n, float t_min,
                                  float t_max, float grid2cell, float* nears,
                                  float* fars) {
    const float cell2grid = (float)(1.0 / grid2cell);
    const float t_grid_step = (float)(grid2cell * 0.5);
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (int64_t i = 0; i < n; ++i) {
        const float* o = origins + 3 * i;
        const float* d = directions + 3 * i;
        float near = -1.f, far = t_max, t = t_min;
        while (t < t_max) {
            float x[3];
            int in_bound = 1;
            for (int a = 0; a < 3; ++a) {
                x[a] = fmaf(t, d[a], o[a]);
                in_bound = in_bound && x[a] >= bbox_min[a] && x[a] <= bbox_max[a];
            }
            if (!in_bound) break;
            int32_t block[3];
            for (int a = 0; a < 3; ++a) block[a] = (int32_t)floorf(x[a] * cell2grid);
            if (lookup(m, block) >= 0) {
                near = near < 0.f ? t : fmaxf(near - t_grid_step, t_min);
                far = fminf(t + t_grid_step, t_max);
            }
            t += t_grid_step;
        }
        nears[i] = near;
        fars[i] = far;
    }
}

/* Both passes of ray_sample (ash/src/sampler.cu:122-214): with `counts` the
 * allocation pass, with `prefix` (inclusive prefix sum of the counts) and the
 * three output arrays the assignment pass. */
void ash_oracle_ray_sample(const ash_oracle_map* m, const float* origins,
                           const float* directions, const float* ray_nears,
                           const float* ray_fars, int64_t n,
                           int64_t max_samples_per_ray, float grid2cell,
                           int64_t* counts, const int64_t* prefix,
                           int64_t* ray_indices, float* t_nears, float* t_fars) {
    const float cell2grid = (float)(1.0 / grid2cell);
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (int64_t i = 0; i < n; ++i) {
        const float* o = origins + 3 * i;
        const float* d = directions + 3 * i;
        const float ray_near = ray_nears[i], ray_far = ray_fars[i];
        const float t_step =
                fmaxf(0.7f, (ray_far - ray_near) / (float)max_samples_per_ray);
        const float t_grid_step = t_step * grid2cell;
        float t = ray_near, t_near = ray_near;
        int64_t local = 0;
        const int64_t start = prefix ? (i == 0 ? 0 : prefix[i - 1]) : 0;
        int moving = 1;
        /* stops as well when a step no longer advances t (range far beyond
         * fp32 resolution), where the reference would not return */
        while (t < ray_far && moving) {
            const float before = t;
            int32_t block[3];
            for (int a = 0; a < 3; ++a) {
                block[a] = (int32_t)floorf(fmaf(t, d[a], o[a]) * cell2grid);
            }
            if (lookup(m, block) < 0) {
                t += t_grid_step;
            } else {
                t += t_step;
                if (prefix) {
                    ray_indices[start + local] = i;
                    t_nears[start + local] = t_near;
                    t_fars[start + local] = t;
                }
                t_near = t;
                ++local;
            }
            moving = t > before;
        }
        if (counts) counts[i] = local;
    }
}

int ash_oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void ash_oracle_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}
