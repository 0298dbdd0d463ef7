// Measurement-only kernels (libfl_calib.so): what this machine's memory system and matrix cores sustain,
// so that the fractions quoted for the attention kernels can be put beside a measured ceiling instead of
// the nominal peak alone.  Nothing here is part of the attention path; libfl_decode_attn.so does not link it.
//   fl_calib_stream_read   128-bit coalesced streaming read of a buffer, plain or non-temporal loads,
//                          one workgroup per contiguous slice (the access pattern of the decode step)
//   fl_calib_stream_read_two  the same bytes as two streams per workgroup, half the buffer apart (K rows and V rows)
//   fl_calib_empty         a kernel that does nothing (launch cadence of back-to-back dependent launches)
//   fl_calib_mfma_f16/f32  register-only loops of v_mfma_f32_32x32x16_f16 / v_mfma_f32_32x32x2_f32
//   fl_calib_coexec        one wave of matrix work and one wave of vector (fma + exp2) work per SIMD, each alone
//                          and both together, on a chosen number of CUs: how far the two pipes overlap, and
//                          what chip-wide load does to the clock
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));

template <int AUX>
__global__ __launch_bounds__(256) void stream_read_kernel(const char *src, uint32_t bytes_per_block, float *sink)
{
    const char *base = src + (size_t)blockIdx.x * bytes_per_block;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(base), 0, (int)bytes_per_block, 0x00020000);
    u32x4 acc = {0u, 0u, 0u, 0u};
    // eight 16-byte loads per lane in flight, 4 KB per instruction and workgroup: the streaming kernel's pattern
    for (uint32_t off = threadIdx.x * 16u; off < bytes_per_block; off += 8u * 4096u) {
        u32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, (uint32_t)u * 4096u, AUX);
#pragma unroll
        for (int u = 0; u < 8; ++u) acc ^= v[u];
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = 1.f; // keeps the loads alive
}

// The decode step's pattern: a workgroup streams TWO slices (its K rows and its V rows, half the buffer apart),
// four 16-byte non-temporal loads per lane in flight on each.
__global__ __launch_bounds__(256) void stream_read_two_kernel(const char *src, uint32_t bytes_per_block, size_t second, float *sink)
{
    const char *base = src + (size_t)blockIdx.x * bytes_per_block;
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(base), 0, (int)bytes_per_block, 0x00020000);
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(base + second), 0, (int)bytes_per_block, 0x00020000);
    u32x4 acc = {0u, 0u, 0u, 0u};
    for (uint32_t off = threadIdx.x * 16u; off < bytes_per_block; off += 4u * 4096u) {
        u32x4 a[4], b[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) a[u] = __builtin_amdgcn_raw_buffer_load_b128(ra, off, (uint32_t)u * 4096u, 2);
#pragma unroll
        for (int u = 0; u < 4; ++u) b[u] = __builtin_amdgcn_raw_buffer_load_b128(rb, off, (uint32_t)u * 4096u, 2);
#pragma unroll
        for (int u = 0; u < 4; ++u) acc ^= a[u] ^ b[u];
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = 1.f;
}

__global__ void empty_kernel() {}

__device__ __forceinline__ float lane_value(uint32_t seed, bool random)
{
    if (!random) return 0.f;
    uint32_t x = seed * 0x9e3779b9u + 0x7f4a7c15u;
    x ^= x >> 16; x *= 0x85ebca6bu; x ^= x >> 13; x *= 0xc2b2ae35u; x ^= x >> 16;
    return (float)(x & 0xffffu) * (4.0f / 65535.0f) - 2.0f; // uniform in [-2, 2]
}

__global__ __launch_bounds__(256) void mfma_f16_kernel(float *sink, int iters, int random)
{
    half8 a[2], b[2];
    const uint32_t id = blockIdx.x * 256u + threadIdx.x;
#pragma unroll
    for (int k = 0; k < 2; ++k)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            a[k][i] = (_Float16)lane_value(id * 32u + k * 8u + i, random != 0);
            b[k][i] = (_Float16)lane_value(id * 32u + 16u + k * 8u + i, random != 0);
        }
    floatx16 c[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) c[j][v] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 4; ++j) c[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[j & 1], b[(j >> 1) & 1], c[j], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) s += c[j][v];
    if (s == 123.456f) sink[0] = s;
}

__global__ __launch_bounds__(256) void mfma_f32_kernel(float *sink, int iters, int random)
{
    const uint32_t id = blockIdx.x * 256u + threadIdx.x;
    float a[2], b[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        a[k] = lane_value(id * 4u + k, random != 0);
        b[k] = lane_value(id * 4u + 2u + k, random != 0);
    }
    floatx16 c[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) c[j][v] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 4; ++j) c[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j & 1], b[(j >> 1) & 1], c[j], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) s += c[j][v];
    if (s == 123.456f) sink[0] = s;
}

// Workgroup of 8 waves, one workgroup per CU (the dynamic LDS size sees to that): waves 0-3 (one per SIMD) run
// chains of 8 dependent v_mfma_f32_32x32x16_f16 (8 x 32 cycles), waves 4-7 blocks of 48 v_fma_f32 + 16 v_exp_f32
// over 16 independent values (the instruction mix of a softmax update).  what: 1 matrix waves only, 2 vector
// waves only, 3 both.
__global__ __launch_bounds__(512) void coexec_kernel(float *sink, int iters, int what)
{
    extern __shared__ char one_workgroup_per_cu[];
    const int wave = threadIdx.x >> 6;
    float r = 0.f;
    if (wave < 4) {
        if (what & 1) {
            half8 a, b;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                a[i] = (_Float16)lane_value(threadIdx.x * 16u + i, true);
                b[i] = (_Float16)lane_value(threadIdx.x * 16u + 8u + i, true);
            }
            floatx16 c;
#pragma unroll
            for (int v = 0; v < 16; ++v) c[v] = 0.f;
            for (int it = 0; it < iters; ++it)
#pragma unroll
                for (int j = 0; j < 8; ++j) c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
#pragma unroll
            for (int v = 0; v < 16; ++v) r += c[v];
        }
    } else if (what & 2) {
        float x[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) x[v] = lane_value(threadIdx.x * 16u + v, true);
        const float s = 0.999f, m = 0.001f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int v = 0; v < 16; ++v) x[v] = __builtin_amdgcn_exp2f(fmaf(x[v], s, m));
#pragma unroll
            for (int k = 0; k < 2; ++k)
#pragma unroll
                for (int v = 0; v < 16; ++v) x[v] = fmaf(x[v], s, m);
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) r += x[v];
    }
    if (r == 123.456f) sink[0] = r;
}

} // namespace

extern "C" {

// Reads `bytes` from src once with `blocks` workgroups of 256 threads, each over one contiguous slice;
// bytes must be a multiple of blocks * 32768.  nontemporal: 0 plain loads, 1 `nt` loads.  Returns a hipError_t.
int fl_calib_stream_read(const void *src, size_t bytes, int blocks, int nontemporal, float *sink, void *stream)
{
    if (!src || !sink || blocks <= 0 || bytes % ((size_t)blocks * 32768u) != 0 || bytes / blocks > 0x7fffffffu) return (int)hipErrorInvalidValue;
    const uint32_t per_block = (uint32_t)(bytes / blocks);
    if (nontemporal)
        hipLaunchKernelGGL(stream_read_kernel<2>, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<const char *>(src), per_block, sink);
    else
        hipLaunchKernelGGL(stream_read_kernel<0>, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<const char *>(src), per_block, sink);
    return (int)hipGetLastError();
}

// Reads `bytes` from src once as two streams: workgroup i reads slice i of the first half and slice i of the second
// half, alternately.  bytes must be a multiple of blocks * 32768.
int fl_calib_stream_read_two(const void *src, size_t bytes, int blocks, float *sink, void *stream)
{
    if (!src || !sink || blocks <= 0 || bytes % ((size_t)blocks * 32768u) != 0 || bytes / 2 / blocks > 0x7fffffffu) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(stream_read_two_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const char *>(src), (uint32_t)(bytes / 2 / blocks), bytes / 2, sink);
    return (int)hipGetLastError();
}

int fl_calib_empty(void *stream)
{
    hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream));
    return (int)hipGetLastError();
}

// blocks workgroups of 4 waves; every wave issues 4 * iters MFMAs.  FLOPs per launch:
//   f16: blocks * 4 * 4 * iters * 2*32*32*16      f32: blocks * 4 * 4 * iters * 2*32*32*2
int fl_calib_mfma(int fp32, int blocks, int iters, int random_operands, float *sink, void *stream)
{
    if (!sink || blocks <= 0 || iters <= 0) return (int)hipErrorInvalidValue;
    if (fp32)
        hipLaunchKernelGGL(mfma_f32_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), sink, iters, random_operands);
    else
        hipLaunchKernelGGL(mfma_f16_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), sink, iters, random_operands);
    return (int)hipGetLastError();
}

// cus workgroups (one per CU); every matrix wave issues 8 * iters MFMAs, every vector wave 64 * iters
// vector instructions.  what: 1 matrix waves, 2 vector waves, 3 both.
int fl_calib_coexec(int what, int cus, int iters, float *sink, void *stream)
{
    if (!sink || cus <= 0 || iters <= 0 || what < 1 || what > 3) return (int)hipErrorInvalidValue;
    const int lds = 96 * 1024;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(coexec_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL(coexec_kernel, dim3(cus), dim3(512), lds, static_cast<hipStream_t>(stream), sink, iters, what);
    return (int)hipGetLastError();
}

} // extern "C"
