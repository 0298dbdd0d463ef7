/*
 * Deterministic synthetic inputs for the decode-attention harness (host only).
 *
 * Counter-based, so element i of tensor t under a seed is a pure function of (seed, t, i):
 *   u  = splitmix64_finalise(seed ^ (t * 0xD6E8FEB86659FD93) ^ i)
 *   u1 = (top 24 bits of u + 1) / 2^24   in (0, 1]
 *   u2 = (next 24 bits of u)   / 2^24    in [0, 1)
 *   z  = sqrt(-2 ln u1) * cos(2 pi u2)   evaluated in double, rounded once to float
 * and, for fp16 tensors, rounded once more to IEEE half (nearest-even, F16C hardware).
 * The same routine fills the buffers handed to the CPU checker and (after a host-to-device
 * copy) to the HIP kernels, which is what "identical seeded inputs" means in the tests.
 *
 * Tensor ids used by the harness: q = 1, k_new = 2, v_new = 3, k_cache = 4, v_cache = 5,
 * per-sequence lengths = 6.
 */
#include <immintrin.h>
#include <math.h>
#include <stddef.h>
#include <stdint.h>

static inline uint64_t mix64(uint64_t x)
{
    uint64_t z = x + 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

static inline uint64_t draw(uint64_t seed, uint64_t tensor_id, uint64_t index)
{
    return mix64(seed ^ (tensor_id * 0xD6E8FEB86659FD93ull) ^ index);
}

static inline float normal_from(uint64_t u)
{
    const double two_pi = 6.283185307179586476925286766559;
    double u1 = (double)((u >> 40) + 1) * (1.0 / 16777216.0);
    double u2 = (double)((u >> 16) & 0xFFFFFFu) * (1.0 / 16777216.0);
    return (float)(sqrt(-2.0 * log(u1)) * cos(two_pi * u2));
}

uint64_t fl_synth_u64(uint64_t seed, uint64_t tensor_id, uint64_t index)
{
    return draw(seed, tensor_id, index);
}

/* dst[i] = scale * N(0,1) for element index0 + i of the tensor */
void fl_synth_normal_f32(float *dst, uint64_t n, uint64_t seed, uint64_t tensor_id,
                         uint64_t index0, float scale, int threads)
{
    if (threads < 1)
        threads = 1;
#pragma omp parallel for num_threads(threads) schedule(static)
    for (int64_t i = 0; i < (int64_t)n; ++i)
        dst[i] = scale * normal_from(draw(seed, tensor_id, index0 + (uint64_t)i));
}

void fl_synth_normal_f16(uint16_t *dst, uint64_t n, uint64_t seed, uint64_t tensor_id,
                         uint64_t index0, float scale, int threads)
{
    if (threads < 1)
        threads = 1;
#pragma omp parallel for num_threads(threads) schedule(static)
    for (int64_t i = 0; i < (int64_t)n; ++i) {
        float v = scale * normal_from(draw(seed, tensor_id, index0 + (uint64_t)i));
        dst[i] = _cvtss_sh(v, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
    }
}

/* dst[i] uniform integer in [lo, hi] (inclusive), by multiply-shift on the top 32 bits */
void fl_synth_uniform_i32(int32_t *dst, uint64_t n, uint64_t seed, uint64_t tensor_id, int32_t lo,
                          int32_t hi)
{
    uint64_t span = (uint64_t)((int64_t)hi - (int64_t)lo + 1);
    for (uint64_t i = 0; i < n; ++i) {
        uint64_t u = draw(seed, tensor_id, i) >> 32;
        dst[i] = (int32_t)((int64_t)lo + (int64_t)((u * span) >> 32));
    }
}
