// Shared device helpers for the gfx950 kernels: storage types, bf16
// conversion, wave64 reductions, and the error codes the C entry points return.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define IMPARO_OK 0
#define IMPARO_BAD_ARGUMENT 1
#define IMPARO_LAUNCH_FAILED 2
#define IMPARO_SCRATCH_TOO_SMALL 3

// dtype codes shared with the Python side
#define IMPARO_F32 0
#define IMPARO_BF16 1

#define WAVE 64

typedef uint16_t bf16_t;   // raw bfloat16 bits

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
    return __uint_as_float(((uint32_t)v) << 16);
}

// round to nearest even; NaN stays NaN (gfx950 converts in hardware, two values per instruction)
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    const __bf16 b = (__bf16)f;
    return *reinterpret_cast<const bf16_t*>(&b);
}

// two values in one register, `lo` in the low half
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const bf16x2_t b = {(__bf16)lo, (__bf16)hi};
    return *reinterpret_cast<const uint32_t*>(&b);
}

template <typename T> __device__ __forceinline__ float load_f32(const T* p, size_t i);
template <> __device__ __forceinline__ float load_f32<float>(const float* p, size_t i) { return p[i]; }
template <> __device__ __forceinline__ float load_f32<bf16_t>(const bf16_t* p, size_t i) { return bf16_to_f32(p[i]); }

template <typename T> __device__ __forceinline__ void store_f32(T* p, size_t i, float v);
template <> __device__ __forceinline__ void store_f32<float>(float* p, size_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void store_f32<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f32_to_bf16(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, WAVE));
    return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// `scratch` holds at least 16 floats of LDS. The order of the additions
// depends only on the block size, never on the data.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = wave_sum(v);
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x / WAVE;
    const int n_waves = (blockDim.x + WAVE - 1) / WAVE;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int i = 0; i < n_waves; ++i) total += scratch[i];
    return total;
}

// ---- what every kernel that norms and rotates a head shares, so that all of them round alike
// The angle is position * inv_freq, the product taken in float64 and rounded to float32; its sine and
// cosine to float32 accuracy. Angles reach 1e5 and more, where a float32 library routine reduces the
// argument with a long integer product (thousands of cycles in which a whole block waits for its table,
// and the routine's code for that case weighs on the small angles too). So everything is done here, in
// float64: the multiple of pi/2 comes off (two constants carry pi/2 to 107 bits; the product with a count
// below 2^17 is exact enough by far), and what is left, at most pi/4, goes into the two power series, cut
// where the next term is below 2e-9 (sine, after x^9) and 2e-10 (cosine, after x^10).
__device__ __forceinline__ void rotation_of(int pos, float inv_freq, float& sn, float& cs) {
    const float theta = (float)((double)pos * (double)inv_freq);
    const double t = (double)theta;
    const double k = rint(t * 0.63661977236758134308);
    double r = fma(-k, 1.57079632679489655800, t);
    r = fma(-k, 6.12323399573676603587e-17, r);
    const double z = r * r;
    double s = fma(z, 1.0 / 362880.0, -1.0 / 5040.0);
    s = fma(z, s, 1.0 / 120.0);
    s = fma(z, s, -1.0 / 6.0);
    s = fma(z * r, s, r);
    double c = fma(z, -1.0 / 3628800.0, 1.0 / 40320.0);
    c = fma(z, c, -1.0 / 720.0);
    c = fma(z, c, 1.0 / 24.0);
    c = fma(z, c, -0.5);
    c = fma(z, c, 1.0);
    const int quarter = (int)((long long)k & 3);
    const float sf = (float)s, cf = (float)c;
    sn = (quarter & 1) ? cf : sf;
    cs = (quarter & 1) ? sf : cf;
    if (quarter == 1 || quarter == 2) cs = -cs;
    if (quarter >= 2) sn = -sn;
}
__device__ __forceinline__ float head_norm_scale(float sum_squares, int head_dim, float eps) {
    return 1.0f / sqrtf(sum_squares / (float)head_dim + eps);
}

// Orders LDS traffic between the lanes of one wave: what any lane wrote before
// is visible to every lane after.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// One per file of kernels: loads that file's code onto the current device (imparo_load_code calls them all).
int imparo_load_code_attention();
int imparo_load_code_attention_mfma();
int imparo_load_code_decode_rows();
int imparo_load_code_elementwise();
int imparo_load_code_gemm();
int imparo_load_code_rope_cache();
int imparo_load_code_sampling();

static inline int launch_status() {
    return hipGetLastError() == hipSuccess ? IMPARO_OK : IMPARO_LAUNCH_FAILED;
}
