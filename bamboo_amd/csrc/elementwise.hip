// Bandwidth-bound kernels of the stage: LayerNorm fwd/bwd, bias-gradient column sums, masked
// softmax fwd/bwd, residual add, MSE head, casts.  One 64-lane wavefront owns one row; lanes
// read 16-byte vectors (lane l takes vector l, l+64, ...) so a wave load covers 1 KiB of
// contiguous memory, rows are kept in registers between the passes of a kernel, and all
// reductions are butterfly shuffles or fixed-order partial sums (no atomics: results are
// reproducible bit for bit).
#include "common.h"

#include <stdarg.h>

#include <atomic>

// ---- error string ------------------------------------------------------------------------
static thread_local char g_err[512] = "";
void bb_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}
extern "C" const char* bb_last_error(void) { return g_err; }
extern "C" int bb_version(void) { return 1; }
static int ln_bwd_static_setup(int dev);
extern "C" int bb_init(void) {
    int dev = 0;
    BB_HIP_CHECK(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    BB_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        bb_set_error("bb_init: device %d is %s, this library is built for gfx950 only", dev, prop.gcnArchName);
        return BB_EHIP;
    }
    return ln_bwd_static_setup(dev);   // so that bb_layernorm_bwd_static has nothing left to set up on this device
}

// =========================================================================================
// LayerNorm
// =========================================================================================
// Row held in registers: lane owns vectors lane, lane+64, ... (IT of them, VEC elements each).
template <typename T, int IT>
__global__ __launch_bounds__(256) void layernorm_fwd_kernel(int kind, int rows, int cols, float eps,
                                                            const T* __restrict__ x, const T* __restrict__ gain,
                                                            const T* __restrict__ shift, T* __restrict__ y,
                                                            float* __restrict__ mean_out, float* __restrict__ rinv_out) {
    constexpr int VEC = Elem<T>::VEC;
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int nvec = cols / VEC;
    const T* xr = x + (int64_t)row * cols;
    float v[IT][VEC];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < IT; ++i) {
        const int c = lane + i * 64;
        if (c < nvec) {
            load_vec(xr + c * VEC, v[i]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) s += v[i][e];
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[i][e] = 0.f;
        }
    }
    const float mean = wave_sum(s) / (float)cols;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < IT; ++i) {
        const int c = lane + i * 64;
        if (c < nvec) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float d = v[i][e] - mean;
                q += d * d;
            }
        }
    }
    q = wave_sum(q);
    float rinv;
    if (kind == BB_LN_ANNOTATED)
        rinv = 1.0f / (sqrtf(q / (float)(cols - 1)) + eps);
    else
        rinv = 1.0f / sqrtf(q / (float)cols + eps);
    if (lane == 0) {
        mean_out[row] = mean;
        rinv_out[row] = rinv;
    }
    T* yr = y + (int64_t)row * cols;
#pragma unroll
    for (int i = 0; i < IT; ++i) {
        const int c = lane + i * 64;
        if (c < nvec) {
            float gv[VEC], bv[VEC], o[VEC];
            load_vec(gain + c * VEC, gv);
            load_vec(shift + c * VEC, bv);
#pragma unroll
            for (int e = 0; e < VEC; ++e) o[e] = gv[e] * ((v[i][e] - mean) * rinv) + bv[e];
            store_vec(yr + c * VEC, o);
        }
    }
}

// N contiguous floats (N a multiple of 4, 16-byte aligned destination)
template <int N> __device__ __forceinline__ void store_f32s(float* dst, const float* v) {
#pragma unroll
    for (int e = 0; e < N; e += 4) *(f32x4*)(dst + e) = f32x4{v[e], v[e + 1], v[e + 2], v[e + 3]};
}

// 16 raw bytes -> VEC floats
__device__ __forceinline__ void unpack16(const u32x4& t, float (&v)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __uint_as_float(t[i]);
}
__device__ __forceinline__ void unpack16(const u32x4& t, float (&v)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(t[i] << 16);
        v[2 * i + 1] = __uint_as_float(t[i] & 0xffff0000u);
    }
}

constexpr int LN_BWD_BLOCKS = 256;
// One block per CU.  A lane keeps five fp32 values per element it owns (gain, two running sums, the normalised input and
// the scaled gradient of the row in flight): up to 16 elements per lane that fits the 128 registers of sixteen waves
// (four per SIMD, to cover the load latency); wider rows take eight or four waves with more registers each instead of
// spilling.
template <typename T, int IT> constexpr int ln_bwd_waves() {
    return IT * Elem<T>::VEC <= 16 ? 16 : IT * Elem<T>::VEC <= 32 ? 8 : 4;
}

// dx per row, dgain/dshift partial sums per block (fixed row->block assignment).
template <typename T, int IT>
__global__ __launch_bounds__((ln_bwd_waves<T, IT>() * 64)) void layernorm_bwd_kernel(int kind, int rows, int cols, float eps,
                                                            const T* __restrict__ x, const T* __restrict__ gain,
                                                            const float* __restrict__ mean_in,
                                                            const float* __restrict__ rinv_in, const T* __restrict__ dy,
                                                            const T* __restrict__ dres, T* __restrict__ dx,
                                                            float* __restrict__ partial, int one_pass) {
    constexpr int VEC = Elem<T>::VEC, LN_BWD_WAVES = ln_bwd_waves<T, IT>();
    extern __shared__ float red[];  // [all waves][2][cols] (one pass) or [3 waves][2][cols] for the cross-wave sum
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nvec = cols / VEC;
    float gv[IT][VEC], dg[IT][VEC], db[IT][VEC];
#pragma unroll
    for (int i = 0; i < IT; ++i) {
        const int c = lane + i * 64;
#pragma unroll
        for (int e = 0; e < VEC; ++e) dg[i][e] = db[i][e] = gv[i][e] = 0.f;
        if (c < nvec) load_vec(gain + c * VEC, gv[i]);
    }
    for (int row = blockIdx.x * LN_BWD_WAVES + wave; row < rows; row += gridDim.x * LN_BWD_WAVES) {
        const float mean = mean_in[row], rinv = rinv_in[row];
        const T* xr = x + (int64_t)row * cols;
        const T* dyr = dy + (int64_t)row * cols;
        float xh[IT][VEC], dyh[IT][VEC];
        u32x4 rres[IT];   // the residual gradient, fetched with the row (16 bytes per vector, unpacked at the end)
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int i = 0; i < IT; ++i) {
            const int c = lane + i * 64;
            if (dres && c < nvec) rres[i] = *(const u32x4*)(dres + (int64_t)row * cols + c * VEC);
        }
#pragma unroll
        for (int i = 0; i < IT; ++i) {
            const int c = lane + i * 64;
            if (c < nvec) {
                float xv[VEC], dv[VEC];
                load_vec(xr + c * VEC, xv);
                load_vec(dyr + c * VEC, dv);
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    xh[i][e] = (xv[e] - mean) * rinv;
                    dyh[i][e] = dv[e] * gv[i][e];
                    dg[i][e] += dv[e] * xh[i][e];
                    db[i][e] += dv[e];
                    s1 += dyh[i][e];
                    s2 += dyh[i][e] * xh[i][e];
                }
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) xh[i][e] = dyh[i][e] = 0.f;
            }
        }
        s1 = wave_sum(s1) / (float)cols;
        s2 = wave_sum(s2);
        float c2;  // coefficient of xh in dx
        if (kind == BB_LN_ANNOTATED) {
            const float sigma = 1.0f / rinv - eps;
            c2 = sigma > 0.f ? s2 / ((float)(cols - 1) * sigma) : 0.f;
        } else {
            c2 = rinv * s2 / (float)cols;
        }
        T* dxr = dx + (int64_t)row * cols;
#pragma unroll
        for (int i = 0; i < IT; ++i) {
            const int c = lane + i * 64;
            if (c < nvec) {
                float o[VEC];
#pragma unroll
                for (int e = 0; e < VEC; ++e) o[e] = rinv * (dyh[i][e] - s1) - xh[i][e] * c2;
                if (dres) {
                    float rv[VEC];
                    unpack16(rres[i], rv);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) o[e] += rv[e];
                }
                store_vec(dxr + c * VEC, o);
            }
        }
    }
    // cross-wave sum.  Where the LDS holds all waves' sums (2 * cols floats each): one barrier, then every
    // thread adds up its share of the 2 * cols outputs over the waves in wave order, and the block's partial row is
    // written by all threads.  Wider rows go three waves per round through three slots (fixed order as well).
    if (one_pass) {
        float* r = red + (int64_t)wave * 2 * cols;
#pragma unroll
        for (int i = 0; i < IT; ++i) {
            const int c = lane + i * 64;
            if (c < nvec) {
                store_f32s<VEC>(r + c * VEC, dg[i]);
                store_f32s<VEC>(r + cols + c * VEC, db[i]);
            }
        }
        __syncthreads();
        float* out = partial + (int64_t)blockIdx.x * 2 * cols;
        for (int t = threadIdx.x; t < 2 * cols; t += LN_BWD_WAVES * 64) {
            float sum = red[t];
#pragma unroll
            for (int w = 1; w < LN_BWD_WAVES; ++w) sum += red[(int64_t)w * 2 * cols + t];
            out[t] = sum;
        }
        return;
    }
    for (int w0 = 1; w0 < LN_BWD_WAVES; w0 += 3) {
        if (wave >= w0 && wave < w0 + 3) {
            float* r = red + (int64_t)(wave - w0) * 2 * cols;
#pragma unroll
            for (int i = 0; i < IT; ++i) {
                const int c = lane + i * 64;
                if (c < nvec) {
                    store_f32s<VEC>(r + c * VEC, dg[i]);
                    store_f32s<VEC>(r + cols + c * VEC, db[i]);
                }
            }
        }
        __syncthreads();
        if (wave == 0) {
            const int nslot = min(3, LN_BWD_WAVES - w0);
            for (int w = 0; w < nslot; ++w) {
                const float* r = red + (int64_t)w * 2 * cols;
#pragma unroll
                for (int i = 0; i < IT; ++i) {
                    const int c = lane + i * 64;
                    if (c < nvec) {
#pragma unroll
                        for (int e = 0; e < VEC; ++e) {
                            dg[i][e] += r[c * VEC + e];
                            db[i][e] += r[cols + c * VEC + e];
                        }
                    }
                }
            }
        }
        __syncthreads();
    }
    if (wave == 0) {
        float* out = partial + (int64_t)blockIdx.x * 2 * cols;
#pragma unroll
        for (int i = 0; i < IT; ++i) {
            const int c = lane + i * 64;
            if (c < nvec) {
                store_f32s<VEC>(out + c * VEC, dg[i]);
                store_f32s<VEC>(out + cols + c * VEC, db[i]);
            }
        }
    }
}

// Sum of partial rows p = first, first + step, ... in that order, eight loads in flight at a time.
__device__ __forceinline__ float sum_partials(const float* __restrict__ src, int first, int step, int nparts, int64_t stride) {
    float s = 0.f;
    int p = first;
    for (; p + 7 * step < nparts; p += 8 * step) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = src[(int64_t)(p + j * step) * stride];
#pragma unroll
        for (int j = 0; j < 8; ++j) s += v[j];
    }
    for (; p < nparts; p += step) s += src[(int64_t)p * stride];
    return s;
}
constexpr int RED_WAVES = 16;

// out[i] += sum_p partial[p * stride + i].  One block owns 64 columns; its sixteen waves sum
// interleaved shares of the partial rows (p = w, w+16, ...) and the sixteen results are combined
// in wave order, so the summation order is fixed by nparts alone.
__global__ __launch_bounds__(RED_WAVES * 64) void reduce_partials_acc_kernel(const float* __restrict__ partial, int nparts,
                                                                             int64_t stride, int n, float* __restrict__ out) {
    __shared__ float red[RED_WAVES][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = blockIdx.x * 64 + lane;
    red[wave][lane] = i < n ? sum_partials(partial + i, wave, RED_WAVES, nparts, stride) : 0.f;
    __syncthreads();
    if (wave == 0 && i < n) {
        float s = red[0][lane];
#pragma unroll
        for (int w = 1; w < RED_WAVES; ++w) s += red[w][lane];
        out[i] += s;
    }
}

// two vectors at once (LayerNorm gain and shift gradients): blockIdx.y picks the half of every
// partial row and the output
__global__ __launch_bounds__(RED_WAVES * 64) void reduce_partials_acc2_kernel(const float* __restrict__ partial, int nparts,
                                                                              int64_t stride, int n, float* __restrict__ out0,
                                                                              float* __restrict__ out1) {
    __shared__ float red[RED_WAVES][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = blockIdx.x * 64 + lane;
    const float* src = partial + (int64_t)blockIdx.y * n;
    float* out = blockIdx.y == 0 ? out0 : out1;
    red[wave][lane] = i < n ? sum_partials(src + i, wave, RED_WAVES, nparts, stride) : 0.f;
    __syncthreads();
    if (wave == 0 && i < n) {
        float s = red[0][lane];
#pragma unroll
        for (int w = 1; w < RED_WAVES; ++w) s += red[w][lane];
        out[i] += s;
    }
}

template <typename T, int IT>
static int ln_fwd_launch(int kind, int rows, int cols, float eps, const void* x, const void* gain, const void* shift,
                         void* y, float* mean, float* rinv, hipStream_t st) {
    hipLaunchKernelGGL((layernorm_fwd_kernel<T, IT>), dim3((rows + 3) / 4), dim3(256), 0, st, kind, rows, cols, eps,
                       (const T*)x, (const T*)gain, (const T*)shift, (T*)y, mean, rinv);
    BB_LAUNCH_CHECK();
    return BB_OK;
}
template <typename T, int IT>
static int ln_bwd_launch(int kind, int rows, int cols, float eps, const void* x, const void* gain, const float* mean,
                         const float* rinv, const void* dy, const void* dres, void* dx, float* ws, hipStream_t st) {
    constexpr int LN_BWD_WAVES = ln_bwd_waves<T, IT>();
    const size_t all = (size_t)LN_BWD_WAVES * 2 * cols * sizeof(float);
    const int one_pass = all <= 128 * 1024;
    const size_t smem = one_pass ? all : (size_t)3 * 2 * cols * sizeof(float);
    auto kern = layernorm_bwd_kernel<T, IT>;
    BB_HIP_CHECK(bb_allow_dynamic_lds((const void*)kern, smem));   // raised on the first (never captured) call that needs it
    hipLaunchKernelGGL(kern, dim3(LN_BWD_BLOCKS), dim3(LN_BWD_WAVES * 64), smem, st, kind, rows, cols, eps, (const T*)x,
                       (const T*)gain, mean, rinv, (const T*)dy, (const T*)dres, (T*)dx, ws, one_pass);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

#define BB_DISPATCH_IT(T, nvec, CALL)                       \
    do {                                                    \
        const int it_ = ((nvec) + 63) / 64;                 \
        if (it_ <= 2) { constexpr int IT = 2; return CALL; }  \
        if (it_ <= 4) { constexpr int IT = 4; return CALL; }  \
        if (it_ <= 8) { constexpr int IT = 8; return CALL; }  \
        if (it_ <= 16) { constexpr int IT = 16; return CALL; } \
    } while (0)

static int check_rowop(const char* name, int dtype, int rows, int cols) {
    BB_REQUIRE(dtype == BB_F32 || dtype == BB_BF16, "%s: bad dtype %d", name, dtype);
    const int vec = dtype == BB_BF16 ? 8 : 4;
    BB_REQUIRE(rows >= 0 && cols > 0, "%s: bad shape %d x %d", name, rows, cols);
    BB_REQUIRE(cols % vec == 0, "%s: cols (%d) must be a multiple of %d", name, cols, vec);
    BB_REQUIRE(cols / vec <= 64 * 16, "%s: cols (%d) too large (max %d)", name, cols, 64 * 16 * vec);
    return BB_OK;
}

extern "C" int bb_layernorm_fwd(int dtype, int kind, int rows, int cols, float eps, const void* x, const void* gain,
                                const void* shift, void* y, float* mean, float* rinv, void* stream) {
    int rc = check_rowop("bb_layernorm_fwd", dtype, rows, cols);
    if (rc) return rc;
    BB_REQUIRE(kind == BB_LN_STANDARD || kind == BB_LN_ANNOTATED, "bb_layernorm_fwd: bad kind %d", kind);
    BB_REQUIRE(x && gain && shift && y && mean && rinv, "bb_layernorm_fwd: null pointer");
    BB_REQUIRE(kind != BB_LN_ANNOTATED || cols > 1, "bb_layernorm_fwd: annotated LayerNorm needs cols > 1");
    if (rows == 0) return BB_OK;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == BB_BF16)
        BB_DISPATCH_IT(bf16, cols / 8, (ln_fwd_launch<bf16, IT>(kind, rows, cols, eps, x, gain, shift, y, mean, rinv, st)));
    else
        BB_DISPATCH_IT(float, cols / 4, (ln_fwd_launch<float, IT>(kind, rows, cols, eps, x, gain, shift, y, mean, rinv, st)));
    return BB_EINVAL;
}

extern "C" int64_t bb_layernorm_bwd_workspace(int cols) { return (int64_t)LN_BWD_BLOCKS * 2 * cols; }

static int ln_bwd_run(const char* who, int dtype, int kind, int rows, int cols, float eps, const void* x, const void* gain,
                      const float* mean, const float* rinv, const void* dy, const void* dres, void* dx, float* dgain,
                      float* dshift, float* workspace, hipStream_t st) {
    int rc = check_rowop(who, dtype, rows, cols);
    if (rc) return rc;
    BB_REQUIRE(kind == BB_LN_STANDARD || kind == BB_LN_ANNOTATED, "%s: bad kind %d", who, kind);
    BB_REQUIRE(x && gain && mean && rinv && dy && dx && dgain && dshift && workspace, "%s: null pointer", who);
    BB_REQUIRE((size_t)3 * 2 * cols * sizeof(float) <= 160 * 1024, "%s: cols (%d) too large (max 6826)", who, cols);
    if (rows == 0) return BB_OK;
    auto finish = [&]() -> int {
        const int nb = (cols + 63) / 64;
        hipLaunchKernelGGL(reduce_partials_acc2_kernel, dim3(nb, 2), dim3(RED_WAVES * 64), 0, st, workspace, LN_BWD_BLOCKS,
                           (int64_t)2 * cols, cols, dgain, dshift);
        BB_LAUNCH_CHECK();
        return BB_OK;
    };
    auto run = [&](auto launch) -> int {
        int r = launch;
        return r ? r : finish();
    };
    if (dtype == BB_BF16)
        BB_DISPATCH_IT(bf16, cols / 8, run(ln_bwd_launch<bf16, IT>(kind, rows, cols, eps, x, gain, mean, rinv, dy, dres, dx, workspace, st)));
    else
        BB_DISPATCH_IT(float, cols / 4, run(ln_bwd_launch<float, IT>(kind, rows, cols, eps, x, gain, mean, rinv, dy, dres, dx, workspace, st)));
    return BB_EINVAL;
}

extern "C" int bb_layernorm_bwd(int dtype, int kind, int rows, int cols, float eps, const void* x, const void* gain,
                                const float* mean, const float* rinv, const void* dy, const void* dres, void* dx,
                                float* dgain, float* dshift, float* workspace, void* stream) {
    return ln_bwd_run("bb_layernorm_bwd", dtype, kind, rows, cols, eps, x, gain, mean, rinv, dy, dres, dx, dgain, dshift, workspace,
                      (hipStream_t)stream);
}

// ---- the same for callers that cannot allocate ---------------------------------------------------------------
// The per-block partial sums of dgain / dshift ([LN_BWD_BLOCKS][2][cols] floats) live in an array that is part of the
// library's device image instead of a caller's workspace.  Every GPU the library runs on holds its own copy (4 MiB,
// until the process ends) at its own address; host code reaches it only through the address that
// hipGetSymbolAddress returns with that device current -- the array's name is no device address on the host.
static __device__ __align__(256) float ln_bwd_static_scratch[LN_BWD_BLOCKS * 2 * BB_LN_BWD_STATIC_MAX_COLS];
constexpr int LN_STATIC_MAX_DEVICES = 64;
// per device: address of its copy, null until set up.  Written once under the mutex (release), read by the entry
// point without it (acquire): a reader that sees the address also sees the set-up that preceded its store.
static std::atomic<float*> g_ln_static_ptr[LN_STATIC_MAX_DEVICES];
static std::mutex g_ln_static_mu;

template <typename T, int IT> static hipError_t ln_bwd_allow_one_pass() {
    // the largest dynamic LDS request the kernel makes for cols <= BB_LN_BWD_STATIC_MAX_COLS: the one-pass layout
    return bb_allow_dynamic_lds((const void*)layernorm_bwd_kernel<T, IT>, 128 * 1024);
}
// once per device, with that device current: the address of the device's copy, and every LDS-limit change the
// entry point could otherwise need on its first call
static int ln_bwd_static_setup(int dev) {
    BB_REQUIRE(dev >= 0 && dev < LN_STATIC_MAX_DEVICES, "bb_layernorm_bwd_static: device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_ln_static_mu);
    if (g_ln_static_ptr[dev].load(std::memory_order_acquire)) return BB_OK;
    float* ptr = nullptr;
    BB_HIP_CHECK(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(ln_bwd_static_scratch)));
    BB_REQUIRE(ptr != nullptr, "bb_layernorm_bwd_static: no address for the scratch array on device %d", dev);
    BB_HIP_CHECK((ln_bwd_allow_one_pass<bf16, 2>()));
    BB_HIP_CHECK((ln_bwd_allow_one_pass<bf16, 4>()));
    BB_HIP_CHECK((ln_bwd_allow_one_pass<bf16, 8>()));
    BB_HIP_CHECK((ln_bwd_allow_one_pass<bf16, 16>()));
    BB_HIP_CHECK((ln_bwd_allow_one_pass<float, 2>()));
    BB_HIP_CHECK((ln_bwd_allow_one_pass<float, 4>()));
    BB_HIP_CHECK((ln_bwd_allow_one_pass<float, 8>()));
    BB_HIP_CHECK((ln_bwd_allow_one_pass<float, 16>()));
    g_ln_static_ptr[dev].store(ptr, std::memory_order_release);
    return BB_OK;
}

extern "C" int bb_layernorm_bwd_static(int dtype, int kind, int rows, int cols, float eps, const void* x, const void* gain,
                                       const float* mean, const float* rinv, const void* dy, const void* dres, void* dx,
                                       float* dgain, float* dshift, void* stream) {
    BB_REQUIRE(cols <= BB_LN_BWD_STATIC_MAX_COLS, "bb_layernorm_bwd_static: cols (%d) beyond the built-in scratch (max %d); "
               "use bb_layernorm_bwd with a workspace", cols, BB_LN_BWD_STATIC_MAX_COLS);
    int dev = 0;
    BB_HIP_CHECK(hipGetDevice(&dev));
    BB_REQUIRE(dev >= 0 && dev < LN_STATIC_MAX_DEVICES, "bb_layernorm_bwd_static: device ordinal %d out of range", dev);
    float* scratch = g_ln_static_ptr[dev].load(std::memory_order_acquire);
    if (!scratch) {    // bb_init was not called on this device: set up now (not under stream capture)
        int rc = ln_bwd_static_setup(dev);
        if (rc) return rc;
        scratch = g_ln_static_ptr[dev].load(std::memory_order_acquire);
    }
    // every block of the kernel writes its whole partial row (zeros where it had no rows) before the reduction
    // reads it: nothing of the previous call's contents is read, so nothing has to be cleared
    return ln_bwd_run("bb_layernorm_bwd_static", dtype, kind, rows, cols, eps, x, gain, mean, rinv, dy, dres, dx, dgain, dshift,
                      scratch, (hipStream_t)stream);
}

// =========================================================================================
// column sums (bias gradient)
// =========================================================================================
constexpr int COLSUM_SPLITS = 64;

template <typename T>
__global__ __launch_bounds__(256) void colsum_partial_kernel(int rows, int cols, const T* __restrict__ x, int64_t ldx,
                                                             float* __restrict__ partial) {
    constexpr int VEC = Elem<T>::VEC;
    __shared__ float red[3][64 * VEC];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c0 = (blockIdx.x * 64 + lane) * VEC;
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
    if (c0 < cols) {
        for (int r = blockIdx.y * 4 + wave; r < rows; r += gridDim.y * 4) {
            float v[VEC];
            load_vec(x + (int64_t)r * ldx + c0, v);
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] += v[e];
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) red[wave - 1][lane * VEC + e] = acc[e];
    }
    __syncthreads();
    if (wave == 0 && c0 < cols) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float a = acc[e];
            for (int w = 0; w < 3; ++w) a += red[w][lane * VEC + e];
            partial[(int64_t)blockIdx.y * cols + c0 + e] = a;
        }
    }
}

extern "C" int64_t bb_colsum_workspace(int cols) { return (int64_t)COLSUM_SPLITS * cols; }

extern "C" int bb_colsum_acc(int dtype, int rows, int cols, const void* x, int64_t ldx, float* out, float* workspace,
                             void* stream) {
    BB_REQUIRE(dtype == BB_F32 || dtype == BB_BF16, "bb_colsum_acc: bad dtype %d", dtype);
    const int vec = dtype == BB_BF16 ? 8 : 4;
    BB_REQUIRE(rows >= 0 && cols > 0 && cols % vec == 0 && ldx % vec == 0 && ldx >= cols,
               "bb_colsum_acc: bad shape rows=%d cols=%d ldx=%lld", rows, cols, (long long)ldx);
    BB_REQUIRE(x && out && workspace, "bb_colsum_acc: null pointer");
    if (rows == 0) return BB_OK;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid((cols + 64 * vec - 1) / (64 * vec), COLSUM_SPLITS);
    if (dtype == BB_BF16)
        hipLaunchKernelGGL(colsum_partial_kernel<bf16>, grid, dim3(256), 0, st, rows, cols, (const bf16*)x, ldx, workspace);
    else
        hipLaunchKernelGGL(colsum_partial_kernel<float>, grid, dim3(256), 0, st, rows, cols, (const float*)x, ldx, workspace);
    hipLaunchKernelGGL(reduce_partials_acc_kernel, dim3((cols + 63) / 64), dim3(RED_WAVES * 64), 0, st, workspace, COLSUM_SPLITS,
                       (int64_t)cols, cols, out);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

// =========================================================================================
// masked softmax (in place)
// =========================================================================================
template <typename T, int IT>
__global__ __launch_bounds__(256) void softmax_fwd_kernel(int mask, int heads, int sq, int sk, int64_t rows,
                                                          T* __restrict__ s, const int32_t* __restrict__ key_len) {
    constexpr int VEC = Elem<T>::VEC;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int q = (int)(row % sq);
    const int b = (int)(row / ((int64_t)heads * sq));
    int limit = sk;  // keep columns < limit
    if (mask == BB_MASK_CAUSAL) limit = min(sk, q + 1);
    else if (mask == BB_MASK_KEY_PADDING) limit = min(sk, key_len[b]);
    const int nvec = sk / VEC;
    T* sr = s + row * sk;
    float v[IT][VEC];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < IT; ++i) {
        const int c = lane + i * 64;
        if (c < nvec) {
            load_vec(sr + c * VEC, v[i]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                if (c * VEC + e >= limit) v[i][e] = -1e9f;
                mx = fmaxf(mx, v[i][e]);
            }
        }
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < IT; ++i) {
        const int c = lane + i * 64;
        if (c < nvec) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                v[i][e] = expf(v[i][e] - mx);
                sum += v[i][e];
            }
        }
    }
    const float inv = 1.0f / wave_sum(sum);
#pragma unroll
    for (int i = 0; i < IT; ++i) {
        const int c = lane + i * 64;
        if (c < nvec) {
            float o[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) o[e] = v[i][e] * inv;
            store_vec(sr + c * VEC, o);
        }
    }
}

template <typename T, int IT>
__global__ __launch_bounds__(256) void softmax_bwd_kernel(int sk, int64_t rows, const T* __restrict__ p,
                                                          T* __restrict__ dp) {
    constexpr int VEC = Elem<T>::VEC;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int nvec = sk / VEC;
    const T* pr = p + row * sk;
    T* dr = dp + row * sk;
    float pv[IT][VEC], dv[IT][VEC];
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < IT; ++i) {
        const int c = lane + i * 64;
        if (c < nvec) {
            load_vec(pr + c * VEC, pv[i]);
            load_vec(dr + c * VEC, dv[i]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) t += pv[i][e] * dv[i][e];
        }
    }
    t = wave_sum(t);
#pragma unroll
    for (int i = 0; i < IT; ++i) {
        const int c = lane + i * 64;
        if (c < nvec) {
            float o[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) o[e] = pv[i][e] * (dv[i][e] - t);
            store_vec(dr + c * VEC, o);
        }
    }
}

template <typename T, int IT>
static int softmax_fwd_launch(int mask, int heads, int sq, int sk, int64_t rows, void* s, const int32_t* kl, hipStream_t st) {
    hipLaunchKernelGGL((softmax_fwd_kernel<T, IT>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, mask, heads, sq, sk,
                       rows, (T*)s, kl);
    BB_LAUNCH_CHECK();
    return BB_OK;
}
template <typename T, int IT>
static int softmax_bwd_launch(int sk, int64_t rows, const void* p, void* dp, hipStream_t st) {
    hipLaunchKernelGGL((softmax_bwd_kernel<T, IT>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, sk, rows,
                       (const T*)p, (T*)dp);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

extern "C" int bb_softmax_fwd(int dtype, int mask, int batch, int heads, int sq, int sk, void* s, const int32_t* key_len,
                              void* stream) {
    int rc = check_rowop("bb_softmax_fwd", dtype, 1, sk);
    if (rc) return rc;
    BB_REQUIRE(mask >= BB_MASK_NONE && mask <= BB_MASK_KEY_PADDING, "bb_softmax_fwd: bad mask %d", mask);
    BB_REQUIRE(mask != BB_MASK_KEY_PADDING || key_len, "bb_softmax_fwd: key_padding mask needs key_len");
    BB_REQUIRE(batch >= 0 && heads >= 0 && sq >= 0 && s, "bb_softmax_fwd: bad arguments");
    const int64_t rows = (int64_t)batch * heads * sq;
    if (rows == 0) return BB_OK;
    BB_REQUIRE((rows + 3) / 4 < (1ll << 31), "bb_softmax_fwd: too many rows");
    hipStream_t st = (hipStream_t)stream;
    if (dtype == BB_BF16)
        BB_DISPATCH_IT(bf16, sk / 8, (softmax_fwd_launch<bf16, IT>(mask, heads, sq, sk, rows, s, key_len, st)));
    else
        BB_DISPATCH_IT(float, sk / 4, (softmax_fwd_launch<float, IT>(mask, heads, sq, sk, rows, s, key_len, st)));
    return BB_EINVAL;
}

extern "C" int bb_softmax_bwd(int dtype, int batch, int heads, int sq, int sk, const void* p, void* dp, void* stream) {
    int rc = check_rowop("bb_softmax_bwd", dtype, 1, sk);
    if (rc) return rc;
    BB_REQUIRE(batch >= 0 && heads >= 0 && sq >= 0 && p && dp, "bb_softmax_bwd: bad arguments");
    const int64_t rows = (int64_t)batch * heads * sq;
    if (rows == 0) return BB_OK;
    BB_REQUIRE((rows + 3) / 4 < (1ll << 31), "bb_softmax_bwd: too many rows");
    hipStream_t st = (hipStream_t)stream;
    if (dtype == BB_BF16)
        BB_DISPATCH_IT(bf16, sk / 8, (softmax_bwd_launch<bf16, IT>(sk, rows, p, dp, st)));
    else
        BB_DISPATCH_IT(float, sk / 4, (softmax_bwd_launch<float, IT>(sk, rows, p, dp, st)));
    return BB_EINVAL;
}

// =========================================================================================
// residual add, cast, fill
// =========================================================================================
template <typename T>
__global__ __launch_bounds__(256) void add_kernel(int64_t nvec, const T* __restrict__ a, const T* __restrict__ b,
                                                  T* __restrict__ out) {
    constexpr int VEC = Elem<T>::VEC;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * 256) {
        float x[VEC], y[VEC];
        load_vec(a + i * VEC, x);
        load_vec(b + i * VEC, y);
#pragma unroll
        for (int e = 0; e < VEC; ++e) x[e] += y[e];
        store_vec(out + i * VEC, x);
    }
}

static unsigned grid_for(int64_t work_items) {
    int64_t b = (work_items + 255) / 256;
    if (b > 256 * 16) b = 256 * 16;  // 16 blocks per CU, grid-stride beyond
    if (b < 1) b = 1;
    return (unsigned)b;
}

extern "C" int bb_residual_add(int dtype, int64_t n, const void* a, const void* b, void* out, void* stream) {
    BB_REQUIRE(dtype == BB_F32 || dtype == BB_BF16, "bb_residual_add: bad dtype %d", dtype);
    const int vec = dtype == BB_BF16 ? 8 : 4;
    BB_REQUIRE(n >= 0 && n % vec == 0, "bb_residual_add: n (%lld) must be a multiple of %d", (long long)n, vec);
    BB_REQUIRE(a && b && out, "bb_residual_add: null pointer");
    if (n == 0) return BB_OK;
    hipStream_t st = (hipStream_t)stream;
    const int64_t nvec = n / vec;
    if (dtype == BB_BF16)
        hipLaunchKernelGGL(add_kernel<bf16>, dim3(grid_for(nvec)), dim3(256), 0, st, nvec, (const bf16*)a, (const bf16*)b, (bf16*)out);
    else
        hipLaunchKernelGGL(add_kernel<float>, dim3(grid_for(nvec)), dim3(256), 0, st, nvec, (const float*)a, (const float*)b, (float*)out);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

// m = sqrt(1 - x): the stand-in "memory" of the reference's DecoderLayerSimple (gpt2.py:31), and its backward
// dx (+)= dm * (-1 / (2 m)).  NaN where x > 1 and an infinite derivative at x = 1, as torch gives them.
template <typename T>
__global__ __launch_bounds__(256) void sqrt1m_fwd_kernel(int64_t nvec, const T* __restrict__ x, T* __restrict__ m) {
    constexpr int VEC = Elem<T>::VEC;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * 256) {
        float v[VEC];
        load_vec(x + i * VEC, v);
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[e] = sqrtf(1.0f - v[e]);
        store_vec(m + i * VEC, v);
    }
}
template <typename T>
__global__ __launch_bounds__(256) void sqrt1m_bwd_kernel(int64_t nvec, const T* __restrict__ dm, const T* __restrict__ m,
                                                         T* __restrict__ dx, int accumulate) {
    constexpr int VEC = Elem<T>::VEC;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * 256) {
        float g[VEC], mv[VEC], acc[VEC];
        load_vec(dm + i * VEC, g);
        load_vec(m + i * VEC, mv);
        if (accumulate) load_vec(dx + i * VEC, acc);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float d = g[e] * (-0.5f / mv[e]);
            acc[e] = accumulate ? acc[e] + d : d;
        }
        store_vec(dx + i * VEC, acc);
    }
}
extern "C" int bb_sqrt_one_minus_fwd(int dtype, int64_t n, const void* x, void* m, void* stream) {
    BB_REQUIRE(dtype == BB_F32 || dtype == BB_BF16, "bb_sqrt_one_minus_fwd: bad dtype %d", dtype);
    const int vec = dtype == BB_BF16 ? 8 : 4;
    BB_REQUIRE(n >= 0 && n % vec == 0, "bb_sqrt_one_minus_fwd: n (%lld) must be a multiple of %d", (long long)n, vec);
    BB_REQUIRE(x && m, "bb_sqrt_one_minus_fwd: null pointer");
    if (n == 0) return BB_OK;
    hipStream_t st = (hipStream_t)stream;
    const int64_t nvec = n / vec;
    if (dtype == BB_BF16)
        hipLaunchKernelGGL(sqrt1m_fwd_kernel<bf16>, dim3(grid_for(nvec)), dim3(256), 0, st, nvec, (const bf16*)x, (bf16*)m);
    else
        hipLaunchKernelGGL(sqrt1m_fwd_kernel<float>, dim3(grid_for(nvec)), dim3(256), 0, st, nvec, (const float*)x, (float*)m);
    BB_LAUNCH_CHECK();
    return BB_OK;
}
extern "C" int bb_sqrt_one_minus_bwd(int dtype, int64_t n, const void* dm, const void* m, void* dx, int accumulate, void* stream) {
    BB_REQUIRE(dtype == BB_F32 || dtype == BB_BF16, "bb_sqrt_one_minus_bwd: bad dtype %d", dtype);
    const int vec = dtype == BB_BF16 ? 8 : 4;
    BB_REQUIRE(n >= 0 && n % vec == 0, "bb_sqrt_one_minus_bwd: n (%lld) must be a multiple of %d", (long long)n, vec);
    BB_REQUIRE(dm && m && dx, "bb_sqrt_one_minus_bwd: null pointer");
    if (n == 0) return BB_OK;
    hipStream_t st = (hipStream_t)stream;
    const int64_t nvec = n / vec;
    if (dtype == BB_BF16)
        hipLaunchKernelGGL(sqrt1m_bwd_kernel<bf16>, dim3(grid_for(nvec)), dim3(256), 0, st, nvec, (const bf16*)dm, (const bf16*)m,
                           (bf16*)dx, accumulate);
    else
        hipLaunchKernelGGL(sqrt1m_bwd_kernel<float>, dim3(grid_for(nvec)), dim3(256), 0, st, nvec, (const float*)dm, (const float*)m,
                           (float*)dx, accumulate);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

// dst = dropout(src) with the decisions of key (k0, k1): element i of the contiguous tensor is kept (and scaled by
// 1 / (1 - p)) when bb_dropout_keep says so.  nn.Dropout in training mode (transformer.py:98-103,125-126,154-158)
// with a mask that is a pure function of (key, i); the same call on a gradient is its backward.
template <typename T>
__global__ __launch_bounds__(256) void dropout_kernel(int64_t nvec, const T* src, T* dst, DropKey key) {
    constexpr int VEC = Elem<T>::VEC;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * 256) {
        float v[VEC];
        load_vec(src + i * VEC, v);
#pragma unroll
        for (int e = 0; e < VEC; e += 2) {   // VEC is even: one hash per two neighbouring elements
            const uint32_t x = key.small ? bb_dropout_pair_bits32(key.k0, key.k1, (uint32_t)(i * VEC + e) >> 1)
                                         : bb_dropout_pair_bits(key.k0, key.k1, (uint64_t)(i * VEC + e) >> 1);
            v[e] = bb_keep_even(x, key.thresh) ? v[e] * key.scale : 0.f;
            v[e + 1] = bb_keep_odd(x, key.thresh) ? v[e + 1] * key.scale : 0.f;
        }
        store_vec(dst + i * VEC, v);
    }
}
extern "C" int bb_dropout_apply(int dtype, int64_t n, const void* src, void* dst, float p, uint32_t k0, uint32_t k1, void* stream) {
    BB_REQUIRE(dtype == BB_F32 || dtype == BB_BF16, "bb_dropout_apply: bad dtype %d", dtype);
    const int vec = dtype == BB_BF16 ? 8 : 4;
    BB_REQUIRE(n >= 0 && n % vec == 0, "bb_dropout_apply: n (%lld) must be a multiple of %d", (long long)n, vec);
    BB_REQUIRE(p >= 0.f && p < 1.f, "bb_dropout_apply: p must be in [0, 1)");
    BB_REQUIRE(src && dst, "bb_dropout_apply: null pointer");
    if (n == 0) return BB_OK;
    const DropKey key = bb_drop_key(p, k0, k1, (uint64_t)n);
    const int64_t nvec = n / vec;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == BB_BF16)
        hipLaunchKernelGGL(dropout_kernel<bf16>, dim3(grid_for(nvec)), dim3(256), 0, st, nvec, (const bf16*)src, (bf16*)dst, key);
    else
        hipLaunchKernelGGL(dropout_kernel<float>, dim3(grid_for(nvec)), dim3(256), 0, st, nvec, (const float*)src, (float*)dst, key);
    BB_LAUNCH_CHECK();
    return BB_OK;
}
extern "C" int bb_dropout_keep_host(float p, uint32_t k0, uint32_t k1, uint64_t index) {
    const DropKey key = bb_drop_key(p, k0, k1, ~0ull);
    return bb_dropout_keep(key.k0, key.k1, key.thresh, index) ? 1 : 0;
}

// y[r] = sum over the columns of row r (the ``lambda x: x.sum(-1)`` that ends the reference's transformer script,
// DeepSpeedExamples/pipeline_parallelism/transformer.py:250) and its backward, dx[r, :] = dy[r].  One wave per row,
// fixed summation order (lane-strided partial sums, then the butterfly).
template <typename T>
__global__ __launch_bounds__(256) void rowsum_fwd_kernel(int rows, int cols, const T* __restrict__ x, T* __restrict__ y) {
    constexpr int VEC = Elem<T>::VEC;
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const T* xr = x + (int64_t)row * cols;
    float s = 0.f;
    for (int c = lane; c < cols / VEC; c += 64) {
        float v[VEC];
        load_vec(xr + c * VEC, v);
#pragma unroll
        for (int e = 0; e < VEC; ++e) s += v[e];
    }
    s = wave_sum(s);
    if (lane == 0) Elem<T>::store(y + row, s);
}
template <typename T>
__global__ __launch_bounds__(256) void rowsum_bwd_kernel(int rows, int cols, const T* __restrict__ dy, T* __restrict__ dx) {
    constexpr int VEC = Elem<T>::VEC;
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float g = Elem<T>::load(dy + row);
    float v[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) v[e] = g;
    T* dr = dx + (int64_t)row * cols;
    for (int c = lane; c < cols / VEC; c += 64) store_vec(dr + c * VEC, v);
}

extern "C" int bb_rowsum_fwd(int dtype, int rows, int cols, const void* x, void* y, void* stream) {
    int rc = check_rowop("bb_rowsum_fwd", dtype, rows, cols);
    if (rc) return rc;
    BB_REQUIRE(x && y, "bb_rowsum_fwd: null pointer");
    if (rows == 0) return BB_OK;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == BB_BF16)
        hipLaunchKernelGGL(rowsum_fwd_kernel<bf16>, dim3((rows + 3) / 4), dim3(256), 0, st, rows, cols, (const bf16*)x, (bf16*)y);
    else
        hipLaunchKernelGGL(rowsum_fwd_kernel<float>, dim3((rows + 3) / 4), dim3(256), 0, st, rows, cols, (const float*)x, (float*)y);
    BB_LAUNCH_CHECK();
    return BB_OK;
}
extern "C" int bb_rowsum_bwd(int dtype, int rows, int cols, const void* dy, void* dx, void* stream) {
    int rc = check_rowop("bb_rowsum_bwd", dtype, rows, cols);
    if (rc) return rc;
    BB_REQUIRE(dy && dx, "bb_rowsum_bwd: null pointer");
    if (rows == 0) return BB_OK;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == BB_BF16)
        hipLaunchKernelGGL(rowsum_bwd_kernel<bf16>, dim3((rows + 3) / 4), dim3(256), 0, st, rows, cols, (const bf16*)dy, (bf16*)dx);
    else
        hipLaunchKernelGGL(rowsum_bwd_kernel<float>, dim3((rows + 3) / 4), dim3(256), 0, st, rows, cols, (const float*)dy, (float*)dx);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

// out = act(x) and, if wanted, dact = act'(x), elementwise (the activation between the two
// feed-forward GEMMs).  dact may alias x: a thread reads its elements before it writes them.
template <typename T, bool DACT>
__global__ __launch_bounds__(256) void act_kernel(int64_t nvec, int act, const T* x, T* __restrict__ out, T* dact) {
    constexpr int VEC = Elem<T>::VEC;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * 256) {
        float v[VEC], a[VEC];
        load_vec(x + i * VEC, v);
#pragma unroll
        for (int e = 0; e < VEC; ++e) a[e] = act_f(v[e], act);
        store_vec(out + i * VEC, a);
        if (DACT) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) a[e] = dact_f(v[e], act);
            store_vec(dact + i * VEC, a);
        }
    }
}

extern "C" int bb_act_fwd(int dtype, int act, int64_t n, const void* x, void* out, void* dact, void* stream) {
    BB_REQUIRE(dtype == BB_F32 || dtype == BB_BF16, "bb_act_fwd: bad dtype %d", dtype);
    BB_REQUIRE(act == BB_ACT_RELU || act == BB_ACT_GELU_TANH, "bb_act_fwd: bad activation %d", act);
    const int vec = dtype == BB_BF16 ? 8 : 4;
    BB_REQUIRE(n >= 0 && n % vec == 0 && (n == 0 || (x && out)), "bb_act_fwd: n (%lld) must be a multiple of %d", (long long)n, vec);
    BB_REQUIRE(out != x && out != dact, "bb_act_fwd: out must not alias x or dact");
    if (n == 0) return BB_OK;
    hipStream_t st = (hipStream_t)stream;
    const int64_t nvec = n / vec;
    dim3 grid(grid_for(nvec)), block(256);
    if (dtype == BB_BF16) {
        if (dact) hipLaunchKernelGGL((act_kernel<bf16, true>), grid, block, 0, st, nvec, act, (const bf16*)x, (bf16*)out, (bf16*)dact);
        else hipLaunchKernelGGL((act_kernel<bf16, false>), grid, block, 0, st, nvec, act, (const bf16*)x, (bf16*)out, (bf16*)nullptr);
    } else {
        if (dact) hipLaunchKernelGGL((act_kernel<float, true>), grid, block, 0, st, nvec, act, (const float*)x, (float*)out, (float*)dact);
        else hipLaunchKernelGGL((act_kernel<float, false>), grid, block, 0, st, nvec, act, (const float*)x, (float*)out, (float*)nullptr);
    }
    BB_LAUNCH_CHECK();
    return BB_OK;
}

template <typename S, typename D>
__global__ __launch_bounds__(256) void cast_kernel(int64_t n, const S* __restrict__ src, D* __restrict__ dst) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
        Elem<D>::store(dst + i, Elem<S>::load(src + i));
}
// same-type copy, 16 bytes per lane (pointers 16-byte aligned); the tail goes element by element
template <typename T>
__global__ __launch_bounds__(256) void copy_kernel(int64_t n, const T* __restrict__ src, T* __restrict__ dst) {
    constexpr int V = 16 / sizeof(T);
    const int64_t nv = n / V;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nv; i += (int64_t)gridDim.x * 256)
        ((f32x4*)dst)[i] = ((const f32x4*)src)[i];
    for (int64_t i = nv * V + (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) dst[i] = src[i];
}

extern "C" int bb_cast(int src_dtype, int dst_dtype, int64_t n, const void* src, void* dst, void* stream) {
    BB_REQUIRE((src_dtype == BB_F32 || src_dtype == BB_BF16) && (dst_dtype == BB_F32 || dst_dtype == BB_BF16),
               "bb_cast: bad dtype");
    BB_REQUIRE(n >= 0 && src && dst, "bb_cast: bad arguments");
    if (n == 0) return BB_OK;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid(grid_for(n)), block(256);
    if (src_dtype == BB_F32 && dst_dtype == BB_BF16)
        hipLaunchKernelGGL((cast_kernel<float, bf16>), grid, block, 0, st, n, (const float*)src, (bf16*)dst);
    else if (src_dtype == BB_BF16 && dst_dtype == BB_F32)
        hipLaunchKernelGGL((cast_kernel<bf16, float>), grid, block, 0, st, n, (const bf16*)src, (float*)dst);
    else if (src_dtype == BB_F32)
        hipLaunchKernelGGL((cast_kernel<float, float>), grid, block, 0, st, n, (const float*)src, (float*)dst);
    else if ((((uintptr_t)src | (uintptr_t)dst) & 15) == 0)
        hipLaunchKernelGGL((copy_kernel<bf16>), dim3(grid_for(n / 8 + 1)), block, 0, st, n, (const bf16*)src, (bf16*)dst);
    else
        hipLaunchKernelGGL((cast_kernel<bf16, bf16>), grid, block, 0, st, n, (const bf16*)src, (bf16*)dst);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

__global__ __launch_bounds__(256) void fill_kernel(float* dst, int64_t n, float value) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) dst[i] = value;
}
extern "C" int bb_fill_f32(float* dst, int64_t n, float value, void* stream) {
    BB_REQUIRE(n >= 0 && (dst || n == 0), "bb_fill_f32: bad arguments");
    if (n == 0) return BB_OK;
    hipLaunchKernelGGL(fill_kernel, dim3(grid_for(n)), dim3(256), 0, (hipStream_t)stream, dst, n, value);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

// =========================================================================================
// MSE head: loss and its gradient in one pass over y
// =========================================================================================
constexpr int MSE_BLOCKS = 1024;

template <typename T>
__global__ __launch_bounds__(256) void mse_partial_kernel(int64_t n, const T* __restrict__ y, const T* __restrict__ t,
                                                          T* __restrict__ dy, float gscale, float* __restrict__ partial) {
    __shared__ float red[4];
    // contiguous slice per block so the summation order is fixed by n alone
    const int64_t per = (n + MSE_BLOCKS - 1) / MSE_BLOCKS;
    const int64_t lo = (int64_t)blockIdx.x * per;
    const int64_t hi = lo + per < n ? lo + per : n;
    float s = 0.f;
    for (int64_t i = lo + threadIdx.x; i < hi; i += 256) {
        const float d = Elem<T>::load(y + i) - Elem<T>::load(t + i);
        s += d * d;
        if (dy) Elem<T>::store(dy + i, gscale * d);
    }
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) partial[blockIdx.x] = (red[0] + red[1]) + (red[2] + red[3]);
}

__global__ __launch_bounds__(64) void mse_final_kernel(const float* __restrict__ partial, float inv_n, int accumulate,
                                                       float* __restrict__ loss) {
    float s = 0.f;
    for (int i = threadIdx.x; i < MSE_BLOCKS; i += 64) s += partial[i];
    s = wave_sum(s);
    if (threadIdx.x == 0) loss[0] = (accumulate ? loss[0] : 0.f) + s * inv_n;
}

extern "C" int64_t bb_mse_workspace(void) { return MSE_BLOCKS; }

extern "C" int bb_mse_fwd_bwd(int dtype, int64_t n, const void* y, const void* target, void* dy, float grad_scale,
                              float* loss_out, int accumulate_loss, float* workspace, void* stream) {
    BB_REQUIRE(dtype == BB_F32 || dtype == BB_BF16, "bb_mse_fwd_bwd: bad dtype %d", dtype);
    BB_REQUIRE(n > 0 && y && target && loss_out && workspace, "bb_mse_fwd_bwd: bad arguments");
    hipStream_t st = (hipStream_t)stream;
    const float gs = grad_scale * 2.0f / (float)n;
    if (dtype == BB_BF16)
        hipLaunchKernelGGL(mse_partial_kernel<bf16>, dim3(MSE_BLOCKS), dim3(256), 0, st, n, (const bf16*)y, (const bf16*)target, (bf16*)dy, gs, workspace);
    else
        hipLaunchKernelGGL(mse_partial_kernel<float>, dim3(MSE_BLOCKS), dim3(256), 0, st, n, (const float*)y, (const float*)target, (float*)dy, gs, workspace);
    hipLaunchKernelGGL(mse_final_kernel, dim3(1), dim3(64), 0, st, workspace, 1.0f / (float)n, accumulate_loss, loss_out);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

// =========================================================================================
// BatchNorm (training mode, per-channel statistics over all rows of an NHWC activation viewed
// as [rows = N*H*W, channels]) and the 3x3 patch gather / scatter of the bottleneck block
// (DeepSpeedExamples/pipeline_parallelism/resnet.py:49-75).
// =========================================================================================
constexpr int BN_SPLITS = 64;
constexpr int BN_WAVES = 16;  // row streams per block; with 64 splits 1024 waves share the rows

// Column partial sums, two per channel, over the rows of one split:
// MODE 0 (forward statistics in one pass): sum (x - p) and sum (x - p)^2 with the pivot p = row 0 of x
//   (mean = p + S1/n, var = S2/n - (S1/n)^2: shifted by a sample of the data the subtraction does not
//   cancel, unlike sum x^2 - n mean^2);
// MODE 2 (backward): sum g and sum g * xhat, with g = dy * (out > 0 if relu_out given).
// A block column covers 64 vectors of a row; where the tensor has at most 32 left for it (256 bf16 channels)
// the two halves of a wave take alternate rows, so no lane idles.  Row streams (waves, or half waves) take rows
// s, s + streams, ...: four rows' loads go out together (the rows of a stage-sized tensor fit in one such round),
// sums are added in row order, halves then waves combined in fixed order.
template <typename T, int MODE>
__global__ __launch_bounds__(BN_WAVES * 64) void bn_colred_kernel(int rows, int cols, const T* __restrict__ x,
                                                        const float* __restrict__ mean, const float* __restrict__ rstd,
                                                        const T* __restrict__ dy, const T* __restrict__ relu_out,
                                                        float* __restrict__ partial) {
    constexpr int VEC = Elem<T>::VEC;
    __shared__ float red[BN_WAVES / 2][2][64 * VEC];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int left = cols / VEC - blockIdx.x * 64;          // vectors of a row from this block column on
    const bool halves = left <= 32;
    const int lv = halves ? (lane & 31) : lane, sub = halves ? (lane >> 5) : 0, nsub = halves ? 2 : 1;
    const int c0 = (blockIdx.x * 64 + lv) * VEC;
    float a0[VEC], a1[VEC], mu[VEC], rs[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) a0[e] = a1[e] = mu[e] = rs[e] = 0.f;
    if (lv < left) {
        if (MODE == 0) {
            load_vec(x + c0, mu);   // the pivot
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                mu[e] = mean[c0 + e];
                rs[e] = rstd[c0 + e];
            }
        }
        const int streams = gridDim.y * BN_WAVES * nsub;
        for (int r = (blockIdx.y * BN_WAVES + wave) * nsub + sub; r < rows; r += 4 * streams) {
            float v[4][VEC], g[4][VEC];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int rj = r + j * streams;
                if (rj < rows) {
                    load_vec(x + (int64_t)rj * cols + c0, v[j]);
                    if (MODE == 2) {
                        load_vec(dy + (int64_t)rj * cols + c0, g[j]);
                        if (relu_out) {
                            float o[VEC];
                            load_vec(relu_out + (int64_t)rj * cols + c0, o);
#pragma unroll
                            for (int e = 0; e < VEC; ++e) g[j][e] = o[e] > 0.f ? g[j][e] : 0.f;
                        }
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (r + j * streams < rows) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        if (MODE == 0) {
                            const float d = v[j][e] - mu[e];
                            a0[e] += d;
                            a1[e] += d * d;
                        } else {
                            a0[e] += g[j][e];
                            a1[e] += g[j][e] * (v[j][e] - mu[e]) * rs[e];
                        }
                    }
                }
            }
        }
    }
    if (halves) {   // both halves end with the sum of the two (a + b = b + a bit for bit)
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            a0[e] += __shfl_xor(a0[e], 32, 64);
            a1[e] += __shfl_xor(a1[e], 32, 64);
        }
    }
    // waves: upper half onto lower half, then every thread adds up one output value over the eight left
    constexpr int HW = BN_WAVES / 2;
    auto put = [&](int slot) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            red[slot][0][lane * VEC + e] = a0[e];
            red[slot][1][lane * VEC + e] = a1[e];
        }
    };
    if (wave >= HW) put(wave - HW);
    __syncthreads();
    if (wave < HW) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            a0[e] += red[wave][0][lane * VEC + e];
            a1[e] += red[wave][1][lane * VEC + e];
        }
    }
    __syncthreads();
    if (wave < HW) put(wave);
    __syncthreads();
    // lanes of the second half hold the same columns as the first where rows were shared between halves
    const int width = halves ? 32 * VEC : 64 * VEC;
    for (int t = threadIdx.x; t < 2 * width; t += BN_WAVES * 64) {
        const int j = t / width, col = t - j * width;
        float sum = red[0][j][col];
#pragma unroll
        for (int w = 1; w < HW; ++w) sum += red[w][j][col];
        const int c = blockIdx.x * 64 * VEC + col;
        if (c < cols) partial[((int64_t)blockIdx.y * 2 + j) * cols + c] = sum;
    }
}

// finish: sums over the BN_SPLITS partial rows in fixed order.
// what 1 (forward): mean = p + S1/n, var = S2/n - (S1/n)^2, rstd = 1/sqrt(var + eps) (+ running stats);
// what 2 (backward): dbeta += s0, dgamma += s1, and the batch means of g and g*xhat for the apply pass
template <typename T>
__global__ __launch_bounds__(256) void bn_finish_kernel(int what, int rows, int cols, float eps, float momentum,
                                                        const float* __restrict__ partial, const T* __restrict__ x,
                                                        float* __restrict__ mean,
                                                        float* __restrict__ rstd, float* __restrict__ run_mean,
                                                        float* __restrict__ run_var, float* __restrict__ dgamma,
                                                        float* __restrict__ dbeta, float* __restrict__ sums) {
    // 32 channels per block, 8 threads per channel: each takes eight consecutive partial rows (one round
    // of loads), the eight sums are added in row order through LDS
    static_assert(BN_SPLITS == 64, "eight row groups of eight");
    __shared__ float red[7][2][32];
    const int col = threadIdx.x & 31, rg = threadIdx.x >> 5;
    const int c = blockIdx.x * 32 + col;
    float s0 = 0.f, s1 = 0.f;
    if (c < cols) {
        float t0[8], t1[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            t0[j] = partial[((int64_t)(rg * 8 + j) * 2) * cols + c];
            t1[j] = partial[((int64_t)(rg * 8 + j) * 2 + 1) * cols + c];
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            s0 += t0[j];
            s1 += t1[j];
        }
    }
    if (rg > 0) {
        red[rg - 1][0][col] = s0;
        red[rg - 1][1][col] = s1;
    }
    __syncthreads();
    if (rg > 0 || c >= cols) return;
    for (int q = 0; q < 7; ++q) {
        s0 += red[q][0][col];
        s1 += red[q][1][col];
    }
    if (what == 1) {
        const float d = s0 / (float)rows;
        const float m = Elem<T>::load(x + c) + d;
        const float var = fmaxf(s1 / (float)rows - d * d, 0.f);
        mean[c] = m;
        rstd[c] = 1.0f / sqrtf(var + eps);
        if (run_mean) {  // nn.BatchNorm2d: running_var uses the unbiased estimate
            run_mean[c] = (1.f - momentum) * run_mean[c] + momentum * m;
            run_var[c] = (1.f - momentum) * run_var[c] + momentum * var * (float)rows / (float)(rows - 1);
        }
    } else {
        dbeta[c] += s0;
        dgamma[c] += s1;
        sums[c] = s0 / (float)rows;
        sums[cols + c] = s1 / (float)rows;
    }
}

// Forward BatchNorm from the strip triples a convolution's GEMM epilogue leaves (per 32 rows and channel: pivot p,
// S1 = sum (x - p), S2 = sum (x - p)^2), statistics and normalisation in ONE launch.  A block owns 64 channels and
// one of gridDim.y row ranges.  Every block first turns the strips of its channels into mean and variance -- a
// strip's mean is p + S1/n and its sum of squared deviations M2 = S2 - S1^2/n (no cancellation: p is a sample of the
// strip); two passes over the triples, which stay in registers (at most 8192 rows): mean = sum n_s mean_s / rows,
// then sum (M2_s + n_s (mean_s - mean)^2) -- lane = channel (256-byte reads), its sixteen waves taking strips w,
// w + 16, ..., the sixteen partial sums added in wave order by every thread (a fixed order, the same in every
// block: all row ranges of a channel normalise with the same bits).  The block of the first row range also writes
// mean, rstd and the running statistics.  Then y = gamma (x - mean) rstd + beta (+ resid) (ReLU) over the block's
// rows, eight lanes per row of the 64 channels (128-byte segments).  The tensor is read once; repeating the small
// strip reduction per row range is cheaper than a launch of its own.
constexpr int BN_STRIP_WAVES = 16, BN_STRIP_MAX = 16;   // 16 * 16 strips = up to 8192 rows
constexpr int BN_FWD_ROW_RANGES = 64;
__global__ __launch_bounds__(BN_STRIP_WAVES * 64) void bn_fwd_strips_kernel(int rows, int cols, float eps, float momentum, int relu,
                                                            const float* __restrict__ strips, const bf16* __restrict__ x,
                                                            const bf16* __restrict__ gamma, const bf16* __restrict__ beta,
                                                            const bf16* __restrict__ resid, bf16* __restrict__ y,
                                                            float* __restrict__ mean, float* __restrict__ rstd,
                                                            float* __restrict__ run_mean, float* __restrict__ run_var) {
    __shared__ float red[2][BN_STRIP_WAVES][64];
    __shared__ float fold[2][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = min(blockIdx.x * 64 + lane, cols - 1);   // lanes past the last channel repeat it and store nothing
    const int nstrips = (rows + 31) / 32;
    // the rows this thread normalises first are fetched now, so that they travel while the statistics are reduced
    const int v8 = (threadIdx.x & 7) * 8, c0 = blockIdx.x * 64 + v8;
    const int per = (rows + gridDim.y - 1) / gridDim.y;
    const int r0 = blockIdx.y * per + (threadIdx.x >> 3), r1 = min(rows, ((int)blockIdx.y + 1) * per);
    const bool first = c0 < cols && r0 < r1;
    float xv[8], rv[8];
    if (first) {
        load_vec(x + (int64_t)r0 * cols + c0, xv);
        if (resid) load_vec(resid + (int64_t)r0 * cols + c0, rv);
    }
    float p[BN_STRIP_MAX], a[BN_STRIP_MAX], b[BN_STRIP_MAX];
#pragma unroll
    for (int j = 0; j < BN_STRIP_MAX; ++j) {
        const int s = min(j * BN_STRIP_WAVES + wave, nstrips - 1);   // clamped: every load is issued, unused ones get n = 0
        const float* t = strips + ((int64_t)s * 3) * cols + c;
        p[j] = t[0];
        a[j] = t[cols];
        b[j] = t[2 * (int64_t)cols];
    }
    float sm = 0.f;
#pragma unroll
    for (int j = 0; j < BN_STRIP_MAX; ++j) {
        const int s = j * BN_STRIP_WAVES + wave;
        const int cnt = s < nstrips ? min(32, rows - s * 32) : 0;
        const float n = (float)cnt, inv = cnt == 32 ? 0.03125f : cnt > 0 ? 1.0f / n : 0.f;
        const float m = p[j] + a[j] * inv;           // the strip's mean
        b[j] = cnt > 0 ? b[j] - a[j] * a[j] * inv : 0.f;   // its sum of squared deviations
        p[j] = m;
        a[j] = n;
        sm += n * m;
    }
    red[0][wave][lane] = sm;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < BN_STRIP_WAVES; ++w) tot += red[0][w][lane];
    const float mu = tot / (float)rows;
    float sq = 0.f;
#pragma unroll
    for (int j = 0; j < BN_STRIP_MAX; ++j) {
        const float d = p[j] - mu;
        sq += b[j] + a[j] * d * d;
    }
    red[1][wave][lane] = sq;
    __syncthreads();
    if (wave == 0) {
        float q = 0.f;
#pragma unroll
        for (int w = 0; w < BN_STRIP_WAVES; ++w) q += red[1][w][lane];
        const float var = fmaxf(q / (float)rows, 0.f);
        const float rs = 1.0f / sqrtf(var + eps);
        const float sc = Elem<bf16>::load(gamma + c) * rs;
        fold[0][lane] = sc;
        fold[1][lane] = Elem<bf16>::load(beta + c) - mu * sc;
        if (blockIdx.y == 0 && blockIdx.x * 64 + lane < cols) {
            mean[c] = mu;
            rstd[c] = rs;
            if (run_mean) {  // nn.BatchNorm2d: running_var uses the unbiased estimate
                run_mean[c] = (1.f - momentum) * run_mean[c] + momentum * mu;
                run_var[c] = (1.f - momentum) * run_var[c] + momentum * var * (float)rows / (float)(rows - 1);
            }
        }
    }
    __syncthreads();
    // normalise the block's rows: thread = (row within a pass of 128, eight channels)
    if (c0 >= cols) return;
    float sc[8], sh[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        sc[e] = fold[0][v8 + e];
        sh[e] = fold[1][v8 + e];
    }
    for (int r = r0; r < r1; r += BN_STRIP_WAVES * 8) {
        const int64_t off = (int64_t)r * cols + c0;
        if (r != r0) {
            load_vec(x + off, xv);
            if (resid) load_vec(resid + off, rv);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) xv[e] = fmaf(xv[e], sc[e], sh[e]);
        if (resid) {
#pragma unroll
            for (int e = 0; e < 8; ++e) xv[e] += rv[e];
        }
        if (relu) {
#pragma unroll
            for (int e = 0; e < 8; ++e) xv[e] = fmaxf(xv[e], 0.f);
        }
        store_vec(y + off, xv);
    }
}

// forward apply: y = gamma * (x - mean) * rstd + beta (+ resid), optional ReLU
template <typename T>
__global__ __launch_bounds__(256) void bn_apply_kernel(int64_t nvec, int cols, int relu, const T* __restrict__ x,
                                                       const float* __restrict__ mean, const float* __restrict__ rstd,
                                                       const T* __restrict__ gamma, const T* __restrict__ beta,
                                                       const T* __restrict__ resid, T* __restrict__ y) {
    constexpr int VEC = Elem<T>::VEC;
    // with a grid stride that is a multiple of the row length a thread stays on its channels:
    // scale and shift are then folded once (y = x * sc + sh), outside the loop
    const int64_t stride = (int64_t)gridDim.x * 256;
    const bool fixed = stride % (cols / VEC) == 0;
    float sc[VEC], sh[VEC];
    auto fold = [&](int c0) {
        float g[VEC], b[VEC];
        load_vec(gamma + c0, g);
        load_vec(beta + c0, b);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            sc[e] = g[e] * rstd[c0 + e];
            sh[e] = b[e] - mean[c0 + e] * sc[e];
        }
    };
    const int64_t first = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (fixed && first < nvec) fold((int)((first * VEC) % cols));
    for (int64_t i = first; i < nvec; i += stride) {
        if (!fixed) fold((int)((i * VEC) % cols));
        float v[VEC];
        load_vec(x + i * VEC, v);
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[e] = fmaf(v[e], sc[e], sh[e]);
        if (resid) {
            float r[VEC];
            load_vec(resid + i * VEC, r);
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[e] += r[e];
        }
        if (relu) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[e] = fmaxf(v[e], 0.f);
        }
        store_vec(y + i * VEC, v);
    }
}

// Backward BatchNorm after the column reduction, finish and apply in ONE launch: a block owns 64 channels and one of
// gridDim.y row ranges.  It first adds up the BN_SPLITS partial rows of its channels (sum g and sum g * xhat; sixteen
// thread groups take four partial rows each, the sixteen sums are added in group order: the same bits in every
// block), folds dx = k g + a x + b per channel (k = gamma rstd, a = -k mean(g xhat) rstd, b = -k mean(g) - a mean)
// -- the block of the first row range also accumulates dgamma and dbeta -- and then applies it to its rows, whose
// first pass was fetched before the reduction.
template <typename T>
__global__ __launch_bounds__(1024) void bn_bwd_finish_apply_kernel(int rows, int cols, const float* __restrict__ partial,
                                                                   const T* __restrict__ x, const float* __restrict__ mean,
                                                                   const float* __restrict__ rstd, const T* __restrict__ gamma,
                                                                   const T* __restrict__ dy, const T* __restrict__ relu_out,
                                                                   T* __restrict__ dx, T* __restrict__ g_out,
                                                                   float* __restrict__ dgamma, float* __restrict__ dbeta) {
    constexpr int VEC = Elem<T>::VEC, LPR = 64 / VEC, RPP = 1024 / LPR;   // lanes per row of the slab, rows per pass
    static_assert(BN_SPLITS == 64, "sixteen groups of four partial rows");
    __shared__ float red[2][16][64];
    __shared__ float fold[3][64];
    const int lane = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int c = min(blockIdx.x * 64 + lane, cols - 1);
    const int vc = (threadIdx.x % LPR) * VEC, c0 = blockIdx.x * 64 + vc;
    const int per = (rows + gridDim.y - 1) / gridDim.y;
    const int r0 = blockIdx.y * per + threadIdx.x / LPR, r1 = min(rows, ((int)blockIdx.y + 1) * per);
    const bool first = c0 < cols && r0 < r1;
    float xv[VEC], gv[VEC], ov[VEC];
    if (first) {
        const int64_t off = (int64_t)r0 * cols + c0;
        load_vec(x + off, xv);
        load_vec(dy + off, gv);
        if (relu_out) load_vec(relu_out + off, ov);
    }
    float t0[4], t1[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        t0[j] = partial[((int64_t)(grp * 4 + j) * 2) * cols + c];
        t1[j] = partial[((int64_t)(grp * 4 + j) * 2 + 1) * cols + c];
    }
    red[0][grp][lane] = (t0[0] + t0[1]) + (t0[2] + t0[3]);
    red[1][grp][lane] = (t1[0] + t1[1]) + (t1[2] + t1[3]);
    __syncthreads();
    if (grp == 0) {
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            s0 += red[0][q][lane];
            s1 += red[1][q][lane];
        }
        const float rs = rstd[c], k = Elem<T>::load(gamma + c) * rs;
        const float ka = -k * (s1 / (float)rows) * rs;
        fold[0][lane] = k;
        fold[1][lane] = ka;
        fold[2][lane] = -k * (s0 / (float)rows) - ka * mean[c];
        if (blockIdx.y == 0 && blockIdx.x * 64 + lane < cols) {
            dbeta[c] += s0;
            dgamma[c] += s1;
        }
    }
    __syncthreads();
    if (c0 >= cols) return;
    float k[VEC], ka[VEC], kb[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        k[e] = fold[0][vc + e];
        ka[e] = fold[1][vc + e];
        kb[e] = fold[2][vc + e];
    }
    for (int r = r0; r < r1; r += RPP) {
        const int64_t off = (int64_t)r * cols + c0;
        if (r != r0) {
            load_vec(x + off, xv);
            load_vec(dy + off, gv);
            if (relu_out) load_vec(relu_out + off, ov);
        }
        if (relu_out) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) gv[e] = ov[e] > 0.f ? gv[e] : 0.f;
        }
        float o[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) o[e] = fmaf(k[e], gv[e], fmaf(ka[e], xv[e], kb[e]));
        store_vec(dx + off, o);
        if (g_out) store_vec(g_out + off, gv);
    }
}

// The same after a kernel that left the sums per 32-row strip (the GEMM or convolution that produced the gradient,
// which has the ReLU mask applied already): a block adds up the strips of its 64 channels -- sixteen thread groups
// take the strips q, q + 16, ... in that order, the sixteen sums are added in group order: the same bits in every
// block -- and applies the folded dx = k g + a x + b to its rows.
template <typename T>
__global__ __launch_bounds__(1024) void bn_bwd_strips_apply_kernel(int rows, int cols, const float* __restrict__ strips,
                                                                   const T* __restrict__ x, const float* __restrict__ mean,
                                                                   const float* __restrict__ rstd, const T* __restrict__ gamma,
                                                                   const T* __restrict__ gin, T* __restrict__ dx,
                                                                   float* __restrict__ dgamma, float* __restrict__ dbeta) {
    constexpr int VEC = Elem<T>::VEC, LPR = 64 / VEC, RPP = 1024 / LPR;
    __shared__ float red[2][16][64];
    __shared__ float fold[3][64];
    const int lane = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int c = min(blockIdx.x * 64 + lane, cols - 1);
    const int vc = (threadIdx.x % LPR) * VEC, c0 = blockIdx.x * 64 + vc;
    const int per = (rows + gridDim.y - 1) / gridDim.y;
    const int r0 = blockIdx.y * per + threadIdx.x / LPR, r1 = min(rows, ((int)blockIdx.y + 1) * per);
    const bool first = c0 < cols && r0 < r1;
    float xv[VEC], gv[VEC];
    if (first) {
        const int64_t off = (int64_t)r0 * cols + c0;
        load_vec(x + off, xv);
        load_vec(gin + off, gv);
    }
    const int nstrips = (rows + 31) / 32;
    float s0 = 0.f, s1 = 0.f;
    for (int q0 = grp; q0 < nstrips; q0 += 16 * 4) {
        // four strips' loads go out together
        float t0[4], t1[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int q = q0 + 16 * j;
            t0[j] = q < nstrips ? strips[((int64_t)q * 2) * cols + c] : 0.f;
            t1[j] = q < nstrips ? strips[((int64_t)q * 2 + 1) * cols + c] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            s0 += t0[j];
            s1 += t1[j];
        }
    }
    red[0][grp][lane] = s0;
    red[1][grp][lane] = s1;
    __syncthreads();
    if (grp == 0) {
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            a0 += red[0][q][lane];
            a1 += red[1][q][lane];
        }
        const float rs = rstd[c], k = Elem<T>::load(gamma + c) * rs;
        const float ka = -k * (a1 / (float)rows) * rs;
        fold[0][lane] = k;
        fold[1][lane] = ka;
        fold[2][lane] = -k * (a0 / (float)rows) - ka * mean[c];
        if (blockIdx.y == 0 && blockIdx.x * 64 + lane < cols) {
            dbeta[c] += a0;
            dgamma[c] += a1;
        }
    }
    __syncthreads();
    if (c0 >= cols) return;
    float k[VEC], ka[VEC], kb[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        k[e] = fold[0][vc + e];
        ka[e] = fold[1][vc + e];
        kb[e] = fold[2][vc + e];
    }
    for (int r = r0; r < r1; r += RPP) {
        const int64_t off = (int64_t)r * cols + c0;
        if (r != r0) {
            load_vec(x + off, xv);
            load_vec(gin + off, gv);
        }
        float o[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) o[e] = fmaf(k[e], gv[e], fmaf(ka[e], xv[e], kb[e]));
        store_vec(dx + off, o);
    }
}

extern "C" int64_t bb_bn_workspace(int cols) { return (int64_t)BN_SPLITS * 2 * cols + 2 * cols; }

static int check_bn(const char* name, int dtype, int rows, int cols) {
    BB_REQUIRE(dtype == BB_F32 || dtype == BB_BF16, "%s: bad dtype %d", name, dtype);
    const int vec = dtype == BB_BF16 ? 8 : 4;
    BB_REQUIRE(rows > 1 && cols > 0 && cols % vec == 0, "%s: bad shape %d x %d", name, rows, cols);
    return BB_OK;
}

extern "C" int bb_batchnorm_fwd(int dtype, int rows, int cols, float eps, float momentum, int relu, const void* x,
                                const void* gamma, const void* beta, const void* resid, void* y, float* mean,
                                float* rstd, float* running_mean, float* running_var, float* workspace, void* stream) {
    int rc = check_bn("bb_batchnorm_fwd", dtype, rows, cols);
    if (rc) return rc;
    BB_REQUIRE(x && gamma && beta && y && mean && rstd && workspace, "bb_batchnorm_fwd: null pointer");
    BB_REQUIRE((running_mean == nullptr) == (running_var == nullptr), "bb_batchnorm_fwd: give both running buffers or none");
    hipStream_t st = (hipStream_t)stream;
    const int vec = dtype == BB_BF16 ? 8 : 4;
    dim3 grid((cols + 64 * vec - 1) / (64 * vec), BN_SPLITS), fgrid((cols + 31) / 32);
    const int64_t nvec = (int64_t)rows * cols / vec;
    const dim3 block(BN_WAVES * 64);
    if (dtype == BB_BF16) {
        hipLaunchKernelGGL((bn_colred_kernel<bf16, 0>), grid, block, 0, st, rows, cols, (const bf16*)x, nullptr, nullptr, nullptr, nullptr, workspace);
        hipLaunchKernelGGL(bn_finish_kernel<bf16>, fgrid, dim3(256), 0, st, 1, rows, cols, eps, momentum, workspace, (const bf16*)x, mean, rstd, running_mean, running_var, nullptr, nullptr, nullptr);
        hipLaunchKernelGGL(bn_apply_kernel<bf16>, dim3(grid_for(nvec)), dim3(256), 0, st, nvec, cols, relu, (const bf16*)x, mean, rstd, (const bf16*)gamma, (const bf16*)beta, (const bf16*)resid, (bf16*)y);
    } else {
        hipLaunchKernelGGL((bn_colred_kernel<float, 0>), grid, block, 0, st, rows, cols, (const float*)x, nullptr, nullptr, nullptr, nullptr, workspace);
        hipLaunchKernelGGL(bn_finish_kernel<float>, fgrid, dim3(256), 0, st, 1, rows, cols, eps, momentum, workspace, (const float*)x, mean, rstd, running_mean, running_var, nullptr, nullptr, nullptr);
        hipLaunchKernelGGL(bn_apply_kernel<float>, dim3(grid_for(nvec)), dim3(256), 0, st, nvec, cols, relu, (const float*)x, mean, rstd, (const float*)gamma, (const float*)beta, (const float*)resid, (float*)y);
    }
    BB_LAUNCH_CHECK();
    return BB_OK;
}

extern "C" int bb_batchnorm_fwd_strips(int dtype, int rows, int cols, float eps, float momentum, int relu, const void* x,
                                       const void* gamma, const void* beta, const void* resid, void* y, float* mean,
                                       float* rstd, float* running_mean, float* running_var, const float* strip_stats,
                                       void* stream) {
    int rc = check_bn("bb_batchnorm_fwd_strips", dtype, rows, cols);
    if (rc) return rc;
    BB_REQUIRE(dtype == BB_BF16, "bb_batchnorm_fwd_strips: bf16 only (the kernels that leave strip statistics are)");
    BB_REQUIRE(x && gamma && beta && y && mean && rstd && strip_stats, "bb_batchnorm_fwd_strips: null pointer");
    BB_REQUIRE(rows <= 32 * BN_STRIP_WAVES * BN_STRIP_MAX, "bb_batchnorm_fwd_strips: at most %d rows", 32 * BN_STRIP_WAVES * BN_STRIP_MAX);
    BB_REQUIRE((running_mean == nullptr) == (running_var == nullptr), "bb_batchnorm_fwd_strips: give both running buffers or none");
    hipStream_t st = (hipStream_t)stream;
    // about one block per CU; wide tensors get fewer row ranges (each repeats the strip reduction of its channels)
    const int slabs = (cols + 63) / 64;
    const int ranges = max(4, min(BN_FWD_ROW_RANGES, 256 / slabs));
    hipLaunchKernelGGL(bn_fwd_strips_kernel, dim3(slabs, ranges), dim3(BN_STRIP_WAVES * 64), 0, st, rows, cols, eps, momentum, relu,
                       strip_stats, (const bf16*)x, (const bf16*)gamma, (const bf16*)beta, (const bf16*)resid, (bf16*)y, mean, rstd,
                       running_mean, running_var);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

extern "C" int bb_batchnorm_bwd(int dtype, int rows, int cols, const void* x, const void* gamma, const float* mean,
                                const float* rstd, const void* dy, const void* relu_out, void* dx, void* g_out,
                                float* dgamma, float* dbeta, float* workspace, void* stream) {
    int rc = check_bn("bb_batchnorm_bwd", dtype, rows, cols);
    if (rc) return rc;
    BB_REQUIRE(x && gamma && mean && rstd && dy && dx && dgamma && dbeta && workspace, "bb_batchnorm_bwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    const int vec = dtype == BB_BF16 ? 8 : 4;
    dim3 grid((cols + 64 * vec - 1) / (64 * vec), BN_SPLITS);
    const int slabs = (cols + 63) / 64;
    dim3 agrid(slabs, max(4, min(64, 256 / slabs)));   // about one block per CU
    const dim3 block(BN_WAVES * 64);
    if (dtype == BB_BF16) {
        hipLaunchKernelGGL((bn_colred_kernel<bf16, 2>), grid, block, 0, st, rows, cols, (const bf16*)x, mean, rstd, (const bf16*)dy, (const bf16*)relu_out, workspace);
        hipLaunchKernelGGL(bn_bwd_finish_apply_kernel<bf16>, agrid, dim3(1024), 0, st, rows, cols, workspace, (const bf16*)x, mean, rstd, (const bf16*)gamma, (const bf16*)dy, (const bf16*)relu_out, (bf16*)dx, (bf16*)g_out, dgamma, dbeta);
    } else {
        hipLaunchKernelGGL((bn_colred_kernel<float, 2>), grid, block, 0, st, rows, cols, (const float*)x, mean, rstd, (const float*)dy, (const float*)relu_out, workspace);
        hipLaunchKernelGGL(bn_bwd_finish_apply_kernel<float>, agrid, dim3(1024), 0, st, rows, cols, workspace, (const float*)x, mean, rstd, (const float*)gamma, (const float*)dy, (const float*)relu_out, (float*)dx, (float*)g_out, dgamma, dbeta);
    }
    BB_LAUNCH_CHECK();
    return BB_OK;
}

// The strip sums where no GEMM epilogue left them (the gradient arrived from another stage, or the shape is not one
// the kernels with the sums take): a wave owns one 32-row strip x 64 columns and adds up exactly as those epilogues
// do -- lane (row group l / 8, eight columns) over its four rows in row order, then the eight row groups in order
// through LDS -- so both ways give the same bits.  Also writes the masked gradient g = dy * (relu_out > 0) (g_out may
// be dy itself).
__global__ __launch_bounds__(256) void bn_bwd_strip_sums_kernel(int rows, int cols, const bf16* x, const float* __restrict__ mean,
                                                                const float* __restrict__ rstd, const bf16* dy, const bf16* relu_out,
                                                                bf16* g_out, float* __restrict__ strips) {
    constexpr int PLD = 68;
    __shared__ float patches[4][16 * PLD];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int strip = blockIdx.y * 4 + wave;
    if (strip * 32 >= rows) return;   // no block-wide barrier below
    float* patch = patches[wave];
    const int prow = lane >> 3, pcol = (lane & 7) * 8;
    const int n = blockIdx.x * 64 + pcol;
    const bool live = n < cols;
    float mu8[8], rs8[8], sg[8], sgx[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) mu8[e] = rs8[e] = sg[e] = sgx[e] = 0.f;
    if (live) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            mu8[e] = mean[n + e];
            rs8[e] = rstd[n + e];
        }
    }
    u32x4 gw[4], xw[4], ow[4];
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int m = strip * 32 + it * 8 + prow;
        gw[it] = xw[it] = ow[it] = u32x4{0u, 0u, 0u, 0u};
        if (live && m < rows) {
            const int64_t off = (int64_t)m * cols + n;
            gw[it] = *(const u32x4*)(dy + off);
            xw[it] = *(const u32x4*)(x + off);
            if (relu_out) ow[it] = *(const u32x4*)(relu_out + off);
        }
    }
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int m = strip * 32 + it * 8 + prow;
        if (live && m < rows) {
            float g[8], xv[8], o[8];
            unpack16(gw[it], g);
            unpack16(xw[it], xv);
            if (relu_out) {
                unpack16(ow[it], o);
#pragma unroll
                for (int e = 0; e < 8; ++e) g[e] = o[e] > 0.f ? g[e] : 0.f;
            }
            if (g_out) store_vec(g_out + (int64_t)m * cols + n, g);
#pragma unroll
            for (int e = 0; e < 8; ++e) bn_bwd_sums_add(g[e], xv[e], mu8[e], rs8[e], sg[e], sgx[e]);
        }
    }
    *(f32x4*)(patch + prow * PLD + pcol) = f32x4{sg[0], sg[1], sg[2], sg[3]};
    *(f32x4*)(patch + prow * PLD + pcol + 4) = f32x4{sg[4], sg[5], sg[6], sg[7]};
    *(f32x4*)(patch + (8 + prow) * PLD + pcol) = f32x4{sgx[0], sgx[1], sgx[2], sgx[3]};
    *(f32x4*)(patch + (8 + prow) * PLD + pcol + 4) = f32x4{sgx[4], sgx[5], sgx[6], sgx[7]};
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the wave's own writes, then its reads: no other wave is involved
    float t0 = 0.f, t1 = 0.f;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        t0 = __fadd_rn(t0, patch[r * PLD + lane]);
        t1 = __fadd_rn(t1, patch[(8 + r) * PLD + lane]);
    }
    const int nc = blockIdx.x * 64 + lane;
    if (nc < cols) {
        strips[((int64_t)strip * 2) * cols + nc] = t0;
        strips[((int64_t)strip * 2 + 1) * cols + nc] = t1;
    }
}

extern "C" int bb_batchnorm_bwd_strip_sums(int dtype, int rows, int cols, const void* x, const float* mean, const float* rstd,
                                           const void* dy, const void* relu_out, void* g_out, float* strips, void* stream) {
    int rc = check_bn("bb_batchnorm_bwd_strip_sums", dtype, rows, cols);
    if (rc) return rc;
    BB_REQUIRE(dtype == BB_BF16, "bb_batchnorm_bwd_strip_sums: bf16 only");
    BB_REQUIRE(x && mean && rstd && dy && strips, "bb_batchnorm_bwd_strip_sums: null pointer");
    BB_REQUIRE(!relu_out || g_out, "bb_batchnorm_bwd_strip_sums: with relu_out the masked gradient needs a place (g_out, may be dy)");
    const int nstrips = (rows + 31) / 32;
    hipLaunchKernelGGL(bn_bwd_strip_sums_kernel, dim3((cols + 63) / 64, (nstrips + 3) / 4), dim3(256), 0, (hipStream_t)stream, rows, cols,
                       (const bf16*)x, mean, rstd, (const bf16*)dy, (const bf16*)relu_out, (bf16*)g_out, strips);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

extern "C" int bb_batchnorm_bwd_strips(int dtype, int rows, int cols, const void* x, const void* gamma, const float* mean,
                                       const float* rstd, const void* g, const float* strips, void* dx, float* dgamma,
                                       float* dbeta, void* stream) {
    int rc = check_bn("bb_batchnorm_bwd_strips", dtype, rows, cols);
    if (rc) return rc;
    BB_REQUIRE(dtype == BB_BF16, "bb_batchnorm_bwd_strips: bf16 only (the kernels that leave the strip sums are)");
    BB_REQUIRE(x && gamma && mean && rstd && g && strips && dx && dgamma && dbeta, "bb_batchnorm_bwd_strips: null pointer");
    const int slabs = (cols + 63) / 64;
    dim3 agrid(slabs, max(4, min(64, 256 / slabs)));   // about one block per CU
    hipLaunchKernelGGL(bn_bwd_strips_apply_kernel<bf16>, agrid, dim3(1024), 0, (hipStream_t)stream, rows, cols, strips, (const bf16*)x,
                       mean, rstd, (const bf16*)gamma, (const bf16*)g, (bf16*)dx, dgamma, dbeta);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

// 3x3, pad 1 patch gather on NHWC with stride s: col[q][tap*C + c] = x[n, s*oy+dy, s*ox+dx, c] (0 outside) for the
// output pixel q = (n, oy, ox) of the [ho, wo] = [(h-1)/s + 1, (w-1)/s + 1] grid, and its adjoint as a gather (every
// input pixel sums the patch entries that referenced it: no atomics)
template <typename T, bool ADJOINT>
__global__ __launch_bounds__(256) void patch3x3_kernel(int n, int h, int w, int c, int s, const T* __restrict__ src,
                                                       T* __restrict__ dst) {
    constexpr int VEC = Elem<T>::VEC;
    const int cv = c / VEC;
    const int ho = (h - 1) / s + 1, wo = (w - 1) / s + 1;
    const int64_t total = ADJOINT ? (int64_t)n * h * w * cv : (int64_t)n * ho * wo * 9 * cv;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        if (!ADJOINT) {
            const int ch = (int)(i % cv) * VEC;
            const int tap = (int)((i / cv) % 9);
            const int64_t q = i / (cv * 9);
            const int ox = (int)(q % wo), oy = (int)((q / wo) % ho);
            const int64_t img = q / ((int64_t)wo * ho);
            const int sy = oy * s + tap / 3 - 1, sx = ox * s + tap % 3 - 1;
            float v[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[e] = 0.f;
            if (sy >= 0 && sy < h && sx >= 0 && sx < w) load_vec(src + ((img * h + sy) * w + sx) * c + ch, v);
            store_vec(dst + (q * 9 + tap) * c + ch, v);
        } else {
            const int ch = (int)(i % cv) * VEC;
            const int64_t p = i / cv;
            const int px = (int)(p % w), py = (int)((p / w) % h);
            const int64_t img = p / ((int64_t)w * h);
            float acc[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
#pragma unroll
            for (int tap = 0; tap < 9; ++tap) {
                // the patch of output pixel (qy, qx) holds x[p] at position tap when s*q + shift(tap) = p
                const int ny = py - (tap / 3 - 1), nx = px - (tap % 3 - 1);
                if (ny >= 0 && nx >= 0 && ny % s == 0 && nx % s == 0 && ny / s < ho && nx / s < wo) {
                    float v[VEC];
                    load_vec(src + (((img * ho + ny / s) * wo + nx / s) * 9 + tap) * c + ch, v);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc[e] += v[e];
                }
            }
            store_vec(dst + p * c + ch, acc);
        }
    }
}

extern "C" int bb_patch3x3_strided(int dtype, int adjoint, int n, int h, int w, int c, int stride, const void* src,
                                   void* dst, void* stream) {
    BB_REQUIRE(dtype == BB_F32 || dtype == BB_BF16, "bb_patch3x3: bad dtype %d", dtype);
    const int vec = dtype == BB_BF16 ? 8 : 4;
    BB_REQUIRE(n > 0 && h > 0 && w > 0 && c > 0 && c % vec == 0 && stride >= 1 && stride <= 4 && src && dst,
               "bb_patch3x3: bad arguments (n=%d h=%d w=%d c=%d stride=%d)", n, h, w, c, stride);
    hipStream_t st = (hipStream_t)stream;
    const int ho = (h - 1) / stride + 1, wo = (w - 1) / stride + 1;
    const int64_t items = adjoint ? (int64_t)n * h * w * (c / vec) : (int64_t)n * ho * wo * 9 * (c / vec);
    dim3 grid(grid_for(items));
    if (dtype == BB_BF16) {
        if (adjoint) hipLaunchKernelGGL((patch3x3_kernel<bf16, true>), grid, dim3(256), 0, st, n, h, w, c, stride, (const bf16*)src, (bf16*)dst);
        else hipLaunchKernelGGL((patch3x3_kernel<bf16, false>), grid, dim3(256), 0, st, n, h, w, c, stride, (const bf16*)src, (bf16*)dst);
    } else {
        if (adjoint) hipLaunchKernelGGL((patch3x3_kernel<float, true>), grid, dim3(256), 0, st, n, h, w, c, stride, (const float*)src, (float*)dst);
        else hipLaunchKernelGGL((patch3x3_kernel<float, false>), grid, dim3(256), 0, st, n, h, w, c, stride, (const float*)src, (float*)dst);
    }
    BB_LAUNCH_CHECK();
    return BB_OK;
}

extern "C" int bb_patch3x3(int dtype, int adjoint, int n, int h, int w, int c, const void* src, void* dst, void* stream) {
    return bb_patch3x3_strided(dtype, adjoint, n, h, w, c, 1, src, dst, stream);
}

// Every s-th pixel of every s-th row of an NHWC tensor (what a 1x1 convolution with stride s reads), and the adjoint
// added in place: dst[n, s*oy, s*ox, :] += src[n, oy, ox, :] (each target is written by one thread).
template <typename T, bool ADJOINT>
__global__ __launch_bounds__(256) void subsample_kernel(int n, int h, int w, int c, int s, const T* __restrict__ src,
                                                        T* __restrict__ dst) {
    constexpr int VEC = Elem<T>::VEC;
    const int cv = c / VEC;
    const int ho = (h - 1) / s + 1, wo = (w - 1) / s + 1;
    const int64_t total = (int64_t)n * ho * wo * cv;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int ch = (int)(i % cv) * VEC;
        const int64_t q = i / cv;
        const int ox = (int)(q % wo), oy = (int)((q / wo) % ho);
        const int64_t img = q / ((int64_t)wo * ho);
        const int64_t p = (img * h + (int64_t)oy * s) * w + (int64_t)ox * s;
        float v[VEC];
        if (!ADJOINT) {
            load_vec(src + p * c + ch, v);
            store_vec(dst + q * c + ch, v);
        } else {
            float d[VEC];
            load_vec(src + q * c + ch, v);
            load_vec(dst + p * c + ch, d);
#pragma unroll
            for (int e = 0; e < VEC; ++e) d[e] += v[e];
            store_vec(dst + p * c + ch, d);
        }
    }
}

extern "C" int bb_subsample(int dtype, int adjoint, int n, int h, int w, int c, int stride, const void* src, void* dst,
                            void* stream) {
    BB_REQUIRE(dtype == BB_F32 || dtype == BB_BF16, "bb_subsample: bad dtype %d", dtype);
    const int vec = dtype == BB_BF16 ? 8 : 4;
    BB_REQUIRE(n > 0 && h > 0 && w > 0 && c > 0 && c % vec == 0 && stride >= 1 && stride <= 4 && src && dst,
               "bb_subsample: bad arguments (n=%d h=%d w=%d c=%d stride=%d)", n, h, w, c, stride);
    hipStream_t st = (hipStream_t)stream;
    const int ho = (h - 1) / stride + 1, wo = (w - 1) / stride + 1;
    dim3 grid(grid_for((int64_t)n * ho * wo * (c / vec)));
    if (dtype == BB_BF16) {
        if (adjoint) hipLaunchKernelGGL((subsample_kernel<bf16, true>), grid, dim3(256), 0, st, n, h, w, c, stride, (const bf16*)src, (bf16*)dst);
        else hipLaunchKernelGGL((subsample_kernel<bf16, false>), grid, dim3(256), 0, st, n, h, w, c, stride, (const bf16*)src, (bf16*)dst);
    } else {
        if (adjoint) hipLaunchKernelGGL((subsample_kernel<float, true>), grid, dim3(256), 0, st, n, h, w, c, stride, (const float*)src, (float*)dst);
        else hipLaunchKernelGGL((subsample_kernel<float, false>), grid, dim3(256), 0, st, n, h, w, c, stride, (const float*)src, (float*)dst);
    }
    BB_LAUNCH_CHECK();
    return BB_OK;
}
