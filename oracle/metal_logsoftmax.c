/* CPU restatement of Tome's fused_log_softmax Metal kernel.  TEST INFRASTRUCTURE ONLY.
 *
 * Follows mlx-impl/model.py:16-66 thread by thread: one 1024-thread group per
 * row, M = 4 contiguous elements per thread per block of 4096, a guarded tail
 * block when V % 4096 != 0, per-thread partials reduced first inside each
 * 32-lane simdgroup and then across the 32 simdgroup results held in
 * `shared[32]`.  Metal does not fix the order inside simd_max / simd_sum; a
 * butterfly (xor-shuffle) order is used here.  exp/log are libm's expf/logf
 * where the kernel uses metal::fast::exp/log (bit-level parity with those is
 * not attainable off Apple hardware; the reference's own bound for this kernel
 * is 5e-3, tests/test_logprob_comparison.py:102).
 *
 * Only tests/ and the cpu_baseline leg of bench.py load this file's library.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define TG 1024      /* threads per threadgroup, model.py:87 */
#define MELEMS 4     /* constexpr int M = 4, model.py:17 */
#define SIMD 32

static inline float bf16_to_f32(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static inline float load_elem(const void* base, int dtype, int64_t i) {
    return dtype == 0 ? ((const float*)base)[i] : bf16_to_f32(((const uint16_t*)base)[i]);
}

static float reduce_tg(float* part, int is_max) {
    /* simd-level butterfly, then the 32 simdgroup results (model.py:38-42, 52-55) */
    float shared[SIMD];
    for (int g = 0; g < TG / SIMD; ++g) {
        float lane[SIMD];
        memcpy(lane, part + g * SIMD, sizeof lane);
        for (int off = SIMD / 2; off > 0; off >>= 1) {
            float nxt[SIMD];
            for (int l = 0; l < SIMD; ++l)
                nxt[l] = is_max ? fmaxf(lane[l], lane[l ^ off]) : lane[l] + lane[l ^ off];
            memcpy(lane, nxt, sizeof lane);
        }
        shared[g] = lane[0];
    }
    for (int off = SIMD / 2; off > 0; off >>= 1) {
        float nxt[SIMD];
        for (int l = 0; l < SIMD; ++l)
            nxt[l] = is_max ? fmaxf(shared[l], shared[l ^ off]) : shared[l] + shared[l ^ off];
        memcpy(shared, nxt, sizeof shared);
    }
    return shared[0];
}

/* dtype: 0 = float32, 1 = bfloat16 (bit patterns).  out has the input's dtype. */
int tome_oracle_metal_log_softmax(const void* logits, void* out, int dtype,
                                  int64_t rows, int64_t V, float temp) {
    if (!logits || !out || rows < 0 || V <= 0 || (dtype != 0 && dtype != 1)) return -1;
    const int block = TG * MELEMS;
    const int64_t full_blocks = V / block;
    const float inv_temp = 1.0f / temp;                       /* model.py:27 */
#pragma omp parallel for schedule(static)
    for (int64_t row = 0; row < rows; ++row) {
        const char* in_row = (const char*)logits + row * V * (dtype == 0 ? 4 : 2);
        char* out_row = (char*)out + row * V * (dtype == 0 ? 4 : 2);
        float part[TG];
        for (int tid = 0; tid < TG; ++tid) {                  /* pass 1, model.py:28-36 */
            float thread_max = -1e30f;
            int64_t offset = (int64_t)tid * MELEMS;
            for (int64_t i = 0; i <= full_blocks; ++i) {
                for (int j = 0; j < MELEMS; ++j)
                    if (offset + j < V)
                        thread_max = fmaxf(thread_max, load_elem(in_row, dtype, offset + j) * inv_temp);
                offset += block;
            }
            part[tid] = thread_max;
        }
        const float row_max = reduce_tg(part, 1);
        for (int tid = 0; tid < TG; ++tid) {                  /* pass 2, model.py:43-50 */
            float sum_exp = 0.0f;
            int64_t offset = (int64_t)tid * MELEMS;
            for (int64_t i = 0; i <= full_blocks; ++i) {
                for (int j = 0; j < MELEMS; ++j)
                    if (offset + j < V)
                        sum_exp += expf(load_elem(in_row, dtype, offset + j) * inv_temp - row_max);
                offset += block;
            }
            part[tid] = sum_exp;
        }
        const float log_sum_exp = logf(reduce_tg(part, 0));   /* model.py:56 */
        const float lse = row_max + log_sum_exp;
        if (dtype == 0) {                                     /* pass 3, model.py:57-65 */
            const float* in = (const float*)in_row;
            float* o = (float*)out_row;
            for (int64_t j = 0; j < V; ++j) o[j] = in[j] * inv_temp - lse;
        } else {
            const uint16_t* in = (const uint16_t*)in_row;
            uint16_t* o = (uint16_t*)out_row;
            const float lse_t = bf16_to_f32(f32_to_bf16(lse));            /* T lse = static_cast<T>(...) */
            for (int64_t j = 0; j < V; ++j) {
                const float z_t = bf16_to_f32(f32_to_bf16(bf16_to_f32(in[j]) * inv_temp));
                o[j] = f32_to_bf16(z_t - lse_t);                          /* subtraction in T */
            }
        }
    }
    return 0;
}

/* node.py:400-404 in scalar C (upcast, divide by temp, max, sum exp, gather), one
 * row per OpenMP task.  Used as the multi-core CPU baseline. */
int tome_oracle_local_compute_logprobs(const void* logits, int dtype, int64_t rows, int64_t V,
                                       const int32_t* ids, float temp, float* out_lp) {
    if (!logits || !ids || !out_lp || rows < 0 || V <= 0 || (dtype != 0 && dtype != 1)) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t row = 0; row < rows; ++row) {
        const char* in_row = (const char*)logits + row * V * (dtype == 0 ? 4 : 2);
        float m = -INFINITY;
        for (int64_t j = 0; j < V; ++j) m = fmaxf(m, load_elem(in_row, dtype, j) / temp);
        /* fp32 sum over 16 interleaved partials, as a vectorised reduction would take it */
        float part[16] = {0};
        for (int64_t j = 0; j < V; ++j) part[j & 15] += expf(load_elem(in_row, dtype, j) / temp - m);
        for (int w = 8; w > 0; w >>= 1)
            for (int l = 0; l < w; ++l) part[l] += part[l + w];
        const float s = part[0];
        out_lp[row] = load_elem(in_row, dtype, ids[row]) / temp - (m + logf(s));
    }
    return 0;
}
