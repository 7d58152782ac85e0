// Shared device/host helpers for the gfx950 kernels of libbamboo_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <mutex>
#include <unordered_map>

#include "../../include/bamboo_hip.h"

typedef __bf16 bf16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define BB_WAVE 64

// ---- error plumbing -------------------------------------------------------------------
void bb_set_error(const char* fmt, ...);

#define BB_REQUIRE(cond, ...)          \
    do {                               \
        if (!(cond)) {                 \
            bb_set_error(__VA_ARGS__); \
            return BB_EINVAL;          \
        }                              \
    } while (0)

#define BB_HIP_CHECK(expr)                                                              \
    do {                                                                                \
        hipError_t e_ = (expr);                                                         \
        if (e_ != hipSuccess) {                                                         \
            bb_set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, \
                         __LINE__);                                                     \
            return BB_EHIP;                                                             \
        }                                                                               \
    } while (0)

#define BB_LAUNCH_CHECK() BB_HIP_CHECK(hipGetLastError())

// Raises a kernel's dynamic-LDS limit to at least `bytes`, once per kernel, size and process.  Callers on several
// threads may arrive together (one thread per pipeline stage, the interpreter lock released during the call): the
// table is guarded, and a kernel counts as configured only after the call has succeeded.
static inline hipError_t bb_allow_dynamic_lds(const void* kern, size_t bytes) {
    if (bytes <= 64 * 1024) return hipSuccess;   // the default limit covers it
    static std::mutex mu;
    static std::unordered_map<uintptr_t, size_t> allowed;   // (kernel, device) -> limit set so far
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const uintptr_t key = (uintptr_t)kern ^ ((uintptr_t)(dev + 1) << 56);
    std::lock_guard<std::mutex> lock(mu);
    auto it = allowed.find(key);
    if (it != allowed.end() && it->second >= bytes) return hipSuccess;
    e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e == hipSuccess) allowed[key] = bytes;
    return e;
}

// ---- scalar conversions -----------------------------------------------------------------
__device__ __forceinline__ float bf2f(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }
__device__ __forceinline__ uint16_t f2bf(float f) {
    return __builtin_bit_cast(uint16_t, (__bf16)f);  // round-to-nearest-even (v_cvt_pk_bf16_f32)
}
// two floats -> two bf16 in one register: a vector conversion, so that it is ONE v_cvt_pk_bf16_f32 (two scalar
// conversions and an OR take three instructions; the rounding is the same)
__device__ __forceinline__ uint32_t pack2bf(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) float f32x2_t;
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
    const f32x2_t f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int VEC = 4;  // elements per 16-byte vector
    __device__ static __forceinline__ float load(const float* p) { return *p; }
    __device__ static __forceinline__ void store(float* p, float v) { *p = v; }
};
template <> struct Elem<bf16> {
    static constexpr int VEC = 8;
    __device__ static __forceinline__ float load(const bf16* p) { return bf2f(*(const uint16_t*)p); }
    __device__ static __forceinline__ void store(bf16* p, float v) { *(uint16_t*)p = f2bf(v); }
};

// 16-byte vector load/store of VEC elements <-> float registers
// One element's share of the backward sums of a batch normalisation (sum g, sum g * xhat with xhat = (x - mean) * rstd),
// in explicitly rounded steps: whichever kernel adds the sums up -- the epilogue of the GEMM that writes g, or the
// stand-alone pass -- the compiler contracts nothing, and with the same order of additions the bits are the same.
__device__ __forceinline__ void bn_bwd_sums_add(float g, float x, float mu, float rs, float& sg, float& sgx) {
    sg = __fadd_rn(sg, g);
    sgx = __fadd_rn(sgx, __fmul_rn(__fmul_rn(g, __fsub_rn(x, mu)), rs));
}
__device__ __forceinline__ void load_vec(const float* p, float (&v)[4]) {
    f32x4 t = *(const f32x4*)p;
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void store_vec(float* p, const float (&v)[4]) {
    f32x4 t = {v[0], v[1], v[2], v[3]};
    *(f32x4*)p = t;
}
__device__ __forceinline__ void load_vec(const bf16* p, float (&v)[8]) {
    u32x4 t = *(const u32x4*)p;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(t[i] << 16);
        v[2 * i + 1] = __uint_as_float(t[i] & 0xffff0000u);
    }
}
__device__ __forceinline__ void store_vec(bf16* p, const float (&v)[8]) {
    u32x4 t;
#pragma unroll
    for (int i = 0; i < 4; ++i) t[i] = pack2bf(v[2 * i], v[2 * i + 1]);
    *(u32x4*)p = t;
}

// ---- wavefront reductions (64 lanes, butterfly: every lane gets the result, fixed order) --
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// ---- activations ------------------------------------------------------------------------
// tanh-GELU: 0.5 x (1 + tanh z) = x * sigmoid(2z), z = k0 (x + k1 x^3).  sigmoid(2z) = 1 / (1 + 2^(x (c0 + c1 x^2))) with
// c0 = -2 k0 log2(e), c1 = c0 k1: three multiply-adds, one v_exp_f32 and one v_rcp_f32 per element (both instructions
// accurate to 1 ulp).  Bare instructions on purpose: a correctly rounded 1 / x expands into a ten-instruction division
// sequence per element, which in a GEMM epilogue that evaluates GELU and its derivative for 128 elements per lane and
// tile is a third of the epilogue's vector work (the matrix cores idle meanwhile).
// GELU'(x) = s + x s (1 - s) dz, dz = d(2z)/dx = 2 k0 (1 + 3 k1 x^2) = d0 + d1 x^2.
#define BB_GELU_C0 (-2.3022081983f)    /* -2 * 0.7978845608 * 1.4426950409 */
#define BB_GELU_C1 (-0.10294323957f)   /* c0 * 0.044715 */
#define BB_GELU_D0 (1.5957691216f)     /* 2 * 0.7978845608 */
#define BB_GELU_D1 (0.21406444882f)    /* 6 * 0.7978845608 * 0.044715 */
__device__ __forceinline__ float sigmoid2z_f(float x, float x2) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * fmaf(BB_GELU_C1, x2, BB_GELU_C0)));
}
__device__ __forceinline__ float gelu_tanh_f(float x) { return x * sigmoid2z_f(x, x * x); }
__device__ __forceinline__ void gelu_dgelu_f(float x, float& a, float& d) {
    const float x2 = x * x, s = sigmoid2z_f(x, x2);
    a = x * s;
    d = fmaf(a * (1.0f - s), fmaf(BB_GELU_D1, x2, BB_GELU_D0), s);
}
__device__ __forceinline__ float dgelu_tanh_f(float x) {
    float a, d;
    gelu_dgelu_f(x, a, d);
    return d;
}
// act(x) and act'(x) together (one sigmoid for both)
__device__ __forceinline__ void act_dact_f(float x, int kind, float& a, float& d) {
    if (kind == BB_ACT_RELU) {
        a = fmaxf(x, 0.0f);
        d = x > 0.0f ? 1.0f : 0.0f;
    } else {
        gelu_dgelu_f(x, a, d);
    }
}
__device__ __forceinline__ float act_f(float x, int kind) {
    return kind == BB_ACT_RELU ? fmaxf(x, 0.0f) : gelu_tanh_f(x);
}
__device__ __forceinline__ float dact_f(float x, int kind) {
    return kind == BB_ACT_RELU ? (x > 0.0f ? 1.0f : 0.0f) : dgelu_tanh_f(x);
}

// ---- dropout -------------------------------------------------------------------------------
// Counter-based keep/drop decision: a pure function of (key, element index), so a redundant forward, a normal
// forward and the backward pass of the same (layer, site, micro-batch) make the same decisions without a mask ever
// being stored.
struct DropKey {
    uint32_t k0, k1, thresh;   // thresh: 16-bit, round(p * 65536); 0: no dropout
    float scale;               // 1 / (1 - p)
    uint32_t small;            // the tensor has fewer than 2^32 elements: indices fit 32-bit arithmetic
};
__host__ __device__ __forceinline__ uint32_t bb_mix32(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352du;
    x ^= x >> 15; x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}
// Dropout decisions as a pure function of (key, element index).  One 32-bit hash serves the two elements 2j and
// 2j + 1 of a tensor: x = mix32(((uint32)j ^ k0) + (k1 ^ rotl(j >> 32, 16))), the low 16 bits decide the even
// element, the high 16 the odd one; an element is kept when its 16 bits are >= thresh = round(p * 65536).  (mix32
// is a full-avalanche finalizer: every output bit depends on every input bit, so the two halves are as good as
// two hashes; p is met to within 1 / 131072.)
__host__ __device__ __forceinline__ uint32_t bb_dropout_pair_bits(uint32_t k0, uint32_t k1, uint64_t pair) {
    const uint32_t hi = (uint32_t)(pair >> 32);
    return bb_mix32(((uint32_t)pair ^ k0) + (k1 ^ ((hi << 16) | (hi >> 16))));
}
// the same for a pair index below 2^32 (its high word is zero)
__host__ __device__ __forceinline__ uint32_t bb_dropout_pair_bits32(uint32_t k0, uint32_t k1, uint32_t pair) {
    return bb_mix32((pair ^ k0) + k1);
}
__host__ __device__ __forceinline__ bool bb_dropout_keep(uint32_t k0, uint32_t k1, uint32_t thresh, uint64_t idx) {
    const uint32_t x = bb_dropout_pair_bits(k0, k1, idx >> 1);
    return ((idx & 1) ? x >> 16 : x & 0xffffu) >= thresh;
}
// both decisions of the pair (even element, odd element) from its hash
__host__ __device__ __forceinline__ bool bb_keep_even(uint32_t x, uint32_t thresh) { return (x & 0xffffu) >= thresh; }
__host__ __device__ __forceinline__ bool bb_keep_odd(uint32_t x, uint32_t thresh) { return (x >> 16) >= thresh; }
static inline DropKey bb_drop_key(float p, uint32_t k0, uint32_t k1, uint64_t numel) {
    DropKey d = {k0, k1, 0u, 1.0f, numel < (1ull << 32) ? 1u : 0u};
    if (p > 0.f) {
        const double t = (double)p * 65536.0;
        d.thresh = t >= 65535.0 ? 65535u : t < 1.0 ? 1u : (uint32_t)(t + 0.5);
        d.scale = 1.0f / (1.0f - p);
    }
    return d;
}

static inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }
