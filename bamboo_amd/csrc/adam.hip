// Fused multi-tensor Adam / AdamW for gfx950.
//
// Replaces the reference's only native kernel on this path,
//   multi_tensor_apply_kernel<TensorListMetadata<4>, AdamFunctor<T>>
//   (csrc/adam/multi_tensor_apply.cuh:32-41, csrc/adam/multi_tensor_adam.cu:28-121),
// bound as multi_tensor_adam(chunk_size, noop_flag, [[g],[p],[m],[v]], lr, b1, b2, eps, step,
// mode, bias_correction, wd) (csrc/adam/fused_adam_frontend.cpp:3-20).
//
// HBM-bound: per parameter 16 B read (g, p, m, v) + 12 B written (p, m, v), + 2 B for the bf16
// compute copy and + 4 B when the gradient is cleared in the same pass.  Tensor descriptors
// travel in the kernel argument block (up to 24 per launch); every 256-thread block owns one
// 4096-element chunk and moves it as 16-byte vectors.
#include "common.h"

#include <math.h>

constexpr int ADAM_MAX_TENSORS = 24;
constexpr int ADAM_CHUNK = 4096;  // elements per block

struct AdamTable {
    float* g[ADAM_MAX_TENSORS];
    float* p[ADAM_MAX_TENSORS];
    float* m[ADAM_MAX_TENSORS];
    float* v[ADAM_MAX_TENSORS];
    bf16* lowp[ADAM_MAX_TENSORS];
    int64_t size[ADAM_MAX_TENSORS];
    int first_block[ADAM_MAX_TENSORS + 1];
    int count;
};

struct AdamHyper {
    float lr, beta1, beta2, eps, bc1, bc2, wd;
    int mode, zero_grad;
    const float* gscale;  // device scalar every gradient is multiplied by first (gradient clipping), or null
};

// The update is written with contraction disabled so that every operation rounds exactly as in
// the scalar statement of the formula (multiply and add are not fused into an FMA).
__device__ __forceinline__ void adam_update(float g, float& p, float& m, float& v, const AdamHyper& h) {
#pragma clang fp contract(off)
    if (h.mode == 0) g = g + h.wd * p;
    m = h.beta1 * m + (1.0f - h.beta1) * g;
    v = h.beta2 * v + (1.0f - h.beta2) * g * g;
    const float mhat = m / h.bc1;
    const float vhat = v / h.bc2;
    const float denom = sqrtf(vhat) + h.eps;
    float update = mhat / denom;
    if (h.mode != 0) update = update + h.wd * p;
    p = p - h.lr * update;
}

__global__ __launch_bounds__(256) void adam_multi_kernel(const AdamTable t, const AdamHyper h) {
    // locate the tensor of this block (at most ADAM_MAX_TENSORS entries, uniform per block)
    int ti = 0;
    while (ti + 1 < t.count && (int)blockIdx.x >= t.first_block[ti + 1]) ++ti;
    const int64_t base = (int64_t)(blockIdx.x - t.first_block[ti]) * ADAM_CHUNK;
    const int64_t n = t.size[ti];
    float* __restrict__ g = t.g[ti];
    float* __restrict__ p = t.p[ti];
    float* __restrict__ m = t.m[ti];
    float* __restrict__ v = t.v[ti];
    bf16* __restrict__ lp = t.lowp[ti];
    // the clipping coefficient (1 where the norm is inside the bound): g * coef rounds as the reference's in-place
    // p.grad.mul_(clip_coef) does, then the update sees the clipped gradient
    const bool scaled = h.gscale != nullptr;
    const float gs = scaled ? *h.gscale : 1.0f;
    // vector path needs the chunk start 16-byte aligned in every array: tensor bases are
    // checked on the host, chunk offsets are multiples of 4096 elements
#pragma unroll
    for (int it = 0; it < ADAM_CHUNK / (256 * 4); ++it) {
        const int64_t i = base + ((int64_t)it * 256 + threadIdx.x) * 4;
        if (i + 4 <= n) {
            f32x4 gv = *(const f32x4*)(g + i), pv = *(const f32x4*)(p + i);
            f32x4 mv = *(const f32x4*)(m + i), vv = *(const f32x4*)(v + i);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float pe = pv[e], me = mv[e], ve = vv[e];
                adam_update(scaled ? gv[e] * gs : gv[e], pe, me, ve, h);
                pv[e] = pe; mv[e] = me; vv[e] = ve;
            }
            *(f32x4*)(p + i) = pv;
            *(f32x4*)(m + i) = mv;
            *(f32x4*)(v + i) = vv;
            if (lp) {
                u32x2 w = {pack2bf(pv[0], pv[1]), pack2bf(pv[2], pv[3])};
                *(u32x2*)(lp + i) = w;
            }
            if (h.zero_grad) {
                f32x4 z = {0.f, 0.f, 0.f, 0.f};
                *(f32x4*)(g + i) = z;
            }
        } else {
            for (int64_t j = i; j < n && j < i + 4; ++j) {
                float pe = p[j], me = m[j], ve = v[j];
                adam_update(scaled ? g[j] * gs : g[j], pe, me, ve, h);
                p[j] = pe; m[j] = me; v[j] = ve;
                if (lp) *(uint16_t*)(lp + j) = f2bf(pe);
                if (h.zero_grad) g[j] = 0.f;
            }
        }
    }
}

// =========================================================================================
// Global gradient norm and clipping coefficient (clip_grad_norm_, deepspeed/runtime/utils.py:259-326,
// called from _take_model_step, deepspeed/runtime/engine.py:1526-1531): total = sqrt(sum over all tensors of
// sum g^2), coef = max_norm / (total + 1e-6), gradients are scaled by it when it is below 1.  Two launches, no
// atomics: every block adds up the squares of one 4096-element chunk (threads in index order, then a fixed
// shuffle / LDS tree) into its slot of the workspace; one block then adds the slots in index order in double
// precision and leaves {total norm, min(coef, 1)} for the Adam kernel to read.
// =========================================================================================
__global__ __launch_bounds__(256) void sumsq_partial_kernel(const AdamTable t, float* __restrict__ partial) {
    int ti = 0;
    while (ti + 1 < t.count && (int)blockIdx.x >= t.first_block[ti + 1]) ++ti;
    const int64_t base = (int64_t)(blockIdx.x - t.first_block[ti]) * ADAM_CHUNK;
    const int64_t n = t.size[ti];
    const float* __restrict__ g = t.g[ti];
    float acc = 0.f;
#pragma unroll
    for (int it = 0; it < ADAM_CHUNK / (256 * 4); ++it) {
        const int64_t i = base + ((int64_t)it * 256 + threadIdx.x) * 4;
        if (i + 4 <= n) {
            const f32x4 gv = *(const f32x4*)(g + i);
            acc += gv[0] * gv[0] + gv[1] * gv[1] + gv[2] * gv[2] + gv[3] * gv[3];
        } else {
            for (int64_t j = i; j < n && j < i + 4; ++j) acc += g[j] * g[j];
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    __shared__ float wsum[4];
    if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) partial[blockIdx.x] = (wsum[0] + wsum[1]) + (wsum[2] + wsum[3]);
}
__global__ __launch_bounds__(256) void clip_coef_kernel(const float* __restrict__ partial, int64_t count, int64_t first,
                                                       float max_norm, float* __restrict__ out, double* __restrict__ carry) {
    // thread t adds slots t, t + 256, ... in that order; the 256 sums are added in thread order by thread 0
    __shared__ double sums[256];
    double acc = 0.0;
    for (int64_t i = threadIdx.x; i < count; i += 256) acc += (double)partial[i];
    sums[threadIdx.x] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double total = first ? 0.0 : *carry;     // several launches of partial sums (more than 24 tensors): carried over
        for (int i = 0; i < 256; ++i) total += sums[i];
        *carry = total;
        const float norm = (float)sqrt(total);
        const float coef = max_norm / (norm + 1e-6f);
        out[0] = norm;
        out[1] = coef < 1.0f ? coef : 1.0f;
    }
}

constexpr int64_t CLIP_WS_HEADER = 4;   // floats in front of the per-block slots: one double carried between launches (+ padding)

extern "C" int64_t bb_grad_clip_workspace(int n_tensors, const int64_t* sizes) {
    int64_t blocks = 0;
    for (int i = 0; i < n_tensors; ++i) blocks += sizes && sizes[i] > 0 ? ceil_div64(sizes[i], ADAM_CHUNK) : 0;
    return CLIP_WS_HEADER + blocks;
}

extern "C" int bb_grad_clip_coef(int n_tensors, void* const* g, const int64_t* sizes, float max_norm, float* out,
                                 float* workspace, void* stream) {
    BB_REQUIRE(n_tensors >= 0 && (n_tensors == 0 || (g && sizes)), "bb_grad_clip_coef: bad tensor table");
    BB_REQUIRE(out && workspace && (uintptr_t)workspace % 8 == 0, "bb_grad_clip_coef: out / workspace missing or workspace not 8-byte aligned");
    BB_REQUIRE(max_norm > 0.f, "bb_grad_clip_coef: max_norm must be positive (got %g)", (double)max_norm);
    hipStream_t st = (hipStream_t)stream;
    double* carry = (double*)workspace;
    float* slots = workspace + CLIP_WS_HEADER;
    int i = 0;
    int64_t first = 1;
    do {
        AdamTable t;
        t.count = 0;
        int64_t blocks = 0;
        while (i < n_tensors && t.count < ADAM_MAX_TENSORS) {
            if (sizes[i] > 0) {
                BB_REQUIRE(g[i] && (uintptr_t)g[i] % 16 == 0, "bb_grad_clip_coef: tensor %d null or not 16-byte aligned", i);
                const int64_t nb = ceil_div64(sizes[i], ADAM_CHUNK);
                if (blocks + nb >= (1ll << 31) - 1) {
                    BB_REQUIRE(t.count > 0, "bb_grad_clip_coef: tensor %d too large", i);
                    break;
                }
                const int c = t.count++;
                t.g[c] = (float*)g[i];
                t.size[c] = sizes[i];
                t.first_block[c] = (int)blocks;
                blocks += nb;
            }
            ++i;
        }
        t.first_block[t.count] = (int)blocks;
        if (blocks > 0) {
            hipLaunchKernelGGL(sumsq_partial_kernel, dim3((unsigned)blocks), dim3(256), 0, st, t, slots);
            BB_LAUNCH_CHECK();
        }
        // also with no blocks at all: out = {0, 1}
        hipLaunchKernelGGL(clip_coef_kernel, dim3(1), dim3(256), 0, st, slots, blocks, first, max_norm, out, carry);
        BB_LAUNCH_CHECK();
        first = 0;
    } while (i < n_tensors);
    return BB_OK;
}

static int adam_multi_run(int n_tensors, void* const* g, void* const* p, void* const* m, void* const* v,
                          void* const* lowp, const int64_t* sizes, float lr, float beta1, float beta2, float eps,
                          int step, int mode, int bias_correction, float weight_decay, int zero_grad,
                          const float* grad_scale, void* stream);

extern "C" int bb_adam_multi(int n_tensors, void* const* g, void* const* p, void* const* m, void* const* v,
                             void* const* lowp, const int64_t* sizes, float lr, float beta1, float beta2, float eps,
                             int step, int mode, int bias_correction, float weight_decay, int zero_grad, void* stream) {
    return adam_multi_run(n_tensors, g, p, m, v, lowp, sizes, lr, beta1, beta2, eps, step, mode, bias_correction, weight_decay,
                          zero_grad, nullptr, stream);
}
extern "C" int bb_adam_multi_scaled(int n_tensors, void* const* g, void* const* p, void* const* m, void* const* v,
                                    void* const* lowp, const int64_t* sizes, float lr, float beta1, float beta2, float eps,
                                    int step, int mode, int bias_correction, float weight_decay, int zero_grad,
                                    const float* grad_scale, void* stream) {
    return adam_multi_run(n_tensors, g, p, m, v, lowp, sizes, lr, beta1, beta2, eps, step, mode, bias_correction, weight_decay,
                          zero_grad, grad_scale, stream);
}

static int adam_multi_run(int n_tensors, void* const* g, void* const* p, void* const* m, void* const* v,
                          void* const* lowp, const int64_t* sizes, float lr, float beta1, float beta2, float eps,
                          int step, int mode, int bias_correction, float weight_decay, int zero_grad,
                          const float* grad_scale, void* stream) {
    BB_REQUIRE(n_tensors >= 0, "bb_adam_multi: negative tensor count");
    BB_REQUIRE(n_tensors == 0 || (g && p && m && v && sizes), "bb_adam_multi: null table");
    BB_REQUIRE(step >= 1, "bb_adam_multi: step must be >= 1 (got %d)", step);
    BB_REQUIRE(mode == 0 || mode == 1, "bb_adam_multi: mode must be 0 (L2) or 1 (AdamW)");
    AdamHyper h;
    h.lr = lr; h.beta1 = beta1; h.beta2 = beta2; h.eps = eps; h.wd = weight_decay;
    h.mode = mode; h.zero_grad = zero_grad;
    h.gscale = grad_scale;
    // bias corrections on the host, as the reference does (multi_tensor_adam.cu:138-142)
    h.bc1 = bias_correction ? (float)(1.0 - pow((double)beta1, (double)step)) : 1.0f;
    h.bc2 = bias_correction ? (float)(1.0 - pow((double)beta2, (double)step)) : 1.0f;
    hipStream_t st = (hipStream_t)stream;
    for (int i = 0; i < n_tensors; ++i) {
        BB_REQUIRE(sizes[i] >= 0, "bb_adam_multi: negative size for tensor %d", i);
        if (sizes[i] == 0) continue;
        BB_REQUIRE(g[i] && p[i] && m[i] && v[i], "bb_adam_multi: null pointer in tensor %d", i);
        BB_REQUIRE(((uintptr_t)g[i] | (uintptr_t)p[i] | (uintptr_t)m[i] | (uintptr_t)v[i]) % 16 == 0,
                   "bb_adam_multi: tensor %d is not 16-byte aligned", i);
        BB_REQUIRE(!(lowp && lowp[i]) || ((uintptr_t)lowp[i] % 8) == 0, "bb_adam_multi: lowp %d is not 8-byte aligned", i);
        BB_REQUIRE(ceil_div64(sizes[i], ADAM_CHUNK) < (1ll << 30), "bb_adam_multi: tensor %d too large", i);
    }
    int i = 0;
    while (i < n_tensors) {
        AdamTable t;
        t.count = 0;
        int64_t blocks = 0;
        while (i < n_tensors && t.count < ADAM_MAX_TENSORS) {
            if (sizes[i] > 0) {
                const int64_t nb = ceil_div64(sizes[i], ADAM_CHUNK);
                if (blocks + nb >= (1ll << 31) - 1) {
                    if (t.count == 0) BB_REQUIRE(false, "bb_adam_multi: tensor %d too large", i);
                    break;
                }
                const int c = t.count++;
                t.g[c] = (float*)g[i]; t.p[c] = (float*)p[i]; t.m[c] = (float*)m[i]; t.v[c] = (float*)v[i];
                t.lowp[c] = lowp ? (bf16*)lowp[i] : nullptr;
                t.size[c] = sizes[i];
                t.first_block[c] = (int)blocks;
                blocks += nb;
            }
            ++i;
        }
        if (t.count == 0) continue;
        t.first_block[t.count] = (int)blocks;
        hipLaunchKernelGGL(adam_multi_kernel, dim3((unsigned)blocks), dim3(256), 0, st, t, h);
        BB_LAUNCH_CHECK();
    }
    return BB_OK;
}
