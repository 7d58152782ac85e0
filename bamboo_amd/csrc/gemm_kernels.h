// Device side of the GEMM family (kernels, operand loaders, fragment readers, epilogues) and the per-kernel launch
// templates; the host-side tile choice and the C entry points are in gemm.hip.
#pragma once
#include "common.h"

#include <utility>

struct GemmArgs {
    const void* A; const void* B; void* C;
    const void* bias; const void* aux_in; void* aux_out; const void* resid;
    float* colsum;  // TN only: += column sums of A over K (the bias gradient of a linear layer)
    int64_t lda, ldb, ldc, ldaux;
    int64_t sA1, sA2, sB1, sB2, sC1, sC2;
    int M, N, K, nb2;
    float alpha;
    int epilogue, act, accumulate, c_f32;
    int tiles_m, tiles_n;
    int conv_h, conv_w, conv_c, conv_row0;  // TN: B is the 3x3 patch matrix of an NHWC tensor (conv_c > 0)
    float* strip_stats;  // [ceil(M / 32)][3][N]: per 32-row strip and output column (pivot, sum (c - pivot), sum (c - pivot)^2)
    DropKey drop;        // dropout on the product after bias and activation, before the residual (thresh 0: none)
};
// Backward statistics of the batch normalisation whose (ReLU'd) output the product is the gradient of: the kernels
// built with STATS = 2 leave, per 32-row strip and column, sum g and sum g * xhat of the stored (masked, bf16-rounded)
// gradient g, with xhat = (x - mean) * rstd of the normalisation's input x ([M, N], rows ldc apart like C).
struct BnBwdArgs {
    const void* x;
    const float* mean;
    const float* rstd;
    float* strips;   // [ceil(M / 32)][2][N]
};
// keep-and-scale factor of element (m, n) of the [M, N] product
__device__ __forceinline__ float drop_factor(const GemmArgs& g, int m, int n) {
    return bb_dropout_keep(g.drop.k0, g.drop.k1, g.drop.thresh, (uint64_t)m * (uint64_t)g.N + (uint64_t)n) ? g.drop.scale : 0.f;
}

// ---- tile order: consecutive logical tiles land on the same XCD (workgroups are dealt
// round-robin over the 8 XCDs, each with a private L2), and walk the output in column
// panels of GROUP_M row-tiles so that an XCD's resident tiles share A rows and B columns.
// logical tile -> (row tile, column tile): column panels of GROUP_M row-tiles
template <int GROUP_M = 8>
__device__ __forceinline__ void panel_coords(int lid, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int width = GROUP_M * tiles_n;
    const int group = lid / width;
    const int first_m = group * GROUP_M;
    const int gsize = min(tiles_m - first_m, GROUP_M);
    tm = first_m + (lid % width) % gsize;
    tn = (lid % width) / gsize;
}
// block id -> logical tile such that XCD x (which receives the block ids = x mod 8) owns the
// contiguous range [x * total / 8, (x + 1) * total / 8) of logical tiles
__device__ __forceinline__ int xcd_contiguous(int bid, int total) {
    const int per = total / 8;
    return (per > 0 && bid < per * 8) ? (bid % 8) * per + bid / 8 : bid;
}
template <int GROUP_M = 8>
__device__ __forceinline__ void tile_coords(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
    panel_coords<GROUP_M>(xcd_contiguous(bid, tiles_m * tiles_n), tiles_m, tiles_n, tm, tn);
}

// Generic scalar epilogue.  T = operand dtype (bias/aux/resid), output fp32 or T.
template <typename T>
__device__ __forceinline__ void epilogue_elem(const GemmArgs& g, int64_t coff, int64_t xoff, int m,
                                              int n, float acc) {
    float v = acc * g.alpha;
    if (g.bias) v += Elem<T>::load((const T*)g.bias + n);
    const int64_t ci = coff + (int64_t)m * g.ldc + n;
    const int64_t xi = xoff + (int64_t)m * g.ldaux + n;
    const float keep = g.drop.thresh ? drop_factor(g, m, n) : 1.0f;
    if (g.epilogue == BB_EPI_ACT) {
        if (g.aux_out) Elem<T>::store((T*)g.aux_out + xi, v);
        v = act_f(v, g.act) * keep;
    } else if (g.epilogue == BB_EPI_DACT) {
        v *= dact_f(Elem<T>::load((const T*)g.aux_in + xi), g.act);
    } else if (g.epilogue == BB_EPI_RESIDUAL) {
        v = v * keep + Elem<T>::load((const T*)g.resid + xi);
    } else if (g.epilogue == BB_EPI_MUL) {
        v *= Elem<T>::load((const T*)g.aux_in + xi);
    } else if (g.epilogue == BB_EPI_MUL_POS) {
        if (g.resid) v += Elem<T>::load((const T*)g.resid + xi);
        v = Elem<T>::load((const T*)g.aux_in + xi) > 0.f ? v : 0.f;
    } else if (g.epilogue == BB_EPI_ACT_DACT) {
        float a, d;
        act_dact_f(v, g.act, a, d);
        Elem<T>::store((T*)g.aux_out + xi, d * keep);
        v = a * keep;
    } else {
        v *= keep;
    }
    if (g.c_f32) {
        float* c = (float*)g.C + ci;
        *c = g.accumulate ? (*c + v) : v;
    } else {
        Elem<T>::store((T*)g.C + ci, v);
    }
}

// Vector epilogue for bf16 operands: 8 consecutive columns of one row (n % 8 == 0, n + 8 <= N).
// (ci, xi: element offsets of (m, n) in C and in the epilogue's operand / second output; b: the bias of the eight
// columns, read by the caller once for all the rows it stores in them)
// The operand the epilogue kind reads beside the product (nullptr: none): the kernels fetch its 16 bytes per lane a
// patch ahead of their use (epilogue_vec8_at<DROP, true>), so that the loads' latency passes under the previous
// patch's work instead of in front of every patch's stores.
__device__ __forceinline__ const bf16* epilogue_operand(const GemmArgs& g) {
    if (g.epilogue == BB_EPI_DACT || g.epilogue == BB_EPI_MUL || g.epilogue == BB_EPI_MUL_POS) return (const bf16*)g.aux_in;
    if (g.epilogue == BB_EPI_RESIDUAL) return (const bf16*)g.resid;
    return nullptr;
}
__device__ __forceinline__ void unpack_bf16x8(const u32x4& t, float (&v)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(t[i] << 16);
        v[2 * i + 1] = __uint_as_float(t[i] & 0xffff0000u);
    }
}
// PRE: `pre` holds the 16 bytes of epilogue_operand(g) at xi (fetched earlier); PRE2: `pre2` those of g.resid at xi where
// BB_EPI_MUL_POS has one
template <bool DROP, bool PRE = false, bool PRE2 = false>
__device__ __forceinline__ void epilogue_vec8_at(const GemmArgs& g, int64_t ci, int64_t xi, int m, int n, float (&v)[8],
                                                 const float (&b)[8], const u32x4& pre = u32x4{0u, 0u, 0u, 0u},
                                                 const u32x4& pre2 = u32x4{0u, 0u, 0u, 0u}) {
    if (g.bias) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += b[e];
    }
    float keep[8];
    const bool drop = DROP && g.drop.thresh != 0;   // DROP = false: no dropout code in the kernel at all
    if (drop) {
        // n is a multiple of 8 and so is N (a condition of the kernels that store eight columns at a time): the index
        // is even, one hash serves two neighbouring columns
        const uint64_t pair = ((uint64_t)m * (uint64_t)g.N + (uint64_t)n) >> 1;
        const uint32_t pair32 = ((uint32_t)m * (uint32_t)g.N + (uint32_t)n) >> 1;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t x = g.drop.small ? bb_dropout_pair_bits32(g.drop.k0, g.drop.k1, pair32 + e)
                                            : bb_dropout_pair_bits(g.drop.k0, g.drop.k1, pair + e);
            keep[2 * e] = bb_keep_even(x, g.drop.thresh) ? g.drop.scale : 0.f;
            keep[2 * e + 1] = bb_keep_odd(x, g.drop.thresh) ? g.drop.scale : 0.f;
        }
    }
    if (g.epilogue == BB_EPI_ACT) {
        if (g.aux_out) store_vec((bf16*)g.aux_out + xi, v);
        // one branch over the kind for the eight elements (inside the element loop the compiler turns it into
        // both evaluations and a select per element)
        if (g.act == BB_ACT_RELU) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = fmaxf(v[e], 0.0f);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = gelu_tanh_f(v[e]);
        }
        if (drop) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] *= keep[e];
        }
    } else if (g.epilogue == BB_EPI_DACT) {
        float u[8];
        if constexpr (PRE) unpack_bf16x8(pre, u);
        else load_vec((const bf16*)g.aux_in + xi, u);
        if (g.act == BB_ACT_RELU) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] *= u[e] > 0.0f ? 1.0f : 0.0f;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] *= dgelu_tanh_f(u[e]);
        }
    } else if (g.epilogue == BB_EPI_RESIDUAL) {
        float r[8];
        if constexpr (PRE) unpack_bf16x8(pre, r);
        else load_vec((const bf16*)g.resid + xi, r);
        if (drop) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] *= keep[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += r[e];
    } else if (g.epilogue == BB_EPI_MUL) {
        float d[8];
        if constexpr (PRE) unpack_bf16x8(pre, d);
        else load_vec((const bf16*)g.aux_in + xi, d);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] *= d[e];
    } else if (g.epilogue == BB_EPI_MUL_POS) {
        float d[8];
        if constexpr (PRE) unpack_bf16x8(pre, d);
        else load_vec((const bf16*)g.aux_in + xi, d);
        if (g.resid) {
            float r[8];
            if constexpr (PRE2) unpack_bf16x8(pre2, r);
            else load_vec((const bf16*)g.resid + xi, r);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] += r[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = d[e] > 0.f ? v[e] : 0.f;
    } else if (g.epilogue == BB_EPI_ACT_DACT) {
        float d[8];
        if (g.act == BB_ACT_RELU) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                d[e] = v[e] > 0.0f ? 1.0f : 0.0f;
                v[e] = fmaxf(v[e], 0.0f);
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) gelu_dgelu_f(v[e], v[e], d[e]);
        }
        if (drop) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                v[e] *= keep[e];
                d[e] *= keep[e];
            }
        }
        store_vec((bf16*)g.aux_out + xi, d);
    } else if (drop) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] *= keep[e];
    }
    if (g.c_f32) {
        float* c = (float*)g.C + ci;
        f32x4 lo = {v[0], v[1], v[2], v[3]}, hi = {v[4], v[5], v[6], v[7]};
        if (g.accumulate) {
            lo += *(const f32x4*)c;
            hi += *(const f32x4*)(c + 4);
        }
        *(f32x4*)c = lo;
        *(f32x4*)(c + 4) = hi;
    } else {
        store_vec((bf16*)g.C + ci, v);
    }
}
template <bool DROP>
__device__ __forceinline__ void epilogue_vec8(const GemmArgs& g, int64_t coff, int m, int n, float (&v)[8]) {
    float b[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (g.bias) load_vec((const bf16*)g.bias + n, b);
    epilogue_vec8_at<DROP>(g, coff + (int64_t)m * g.ldc + n, coff + (int64_t)m * g.ldaux + n, m, n, v, b);
}

template <typename F, int... Is> __device__ __forceinline__ void static_for(F&& f, std::integer_sequence<int, Is...>) {
    (f(std::integral_constant<int, Is>{}), ...);
}

// =========================================================================================
// bf16 kernel
// =========================================================================================
__device__ __forceinline__ int swz(int row) {
    return ((row >> 1) & 7) ^ ((row & 1) << 2) ^ ((row >> 4) & 7);
}

// Loader of one operand tile: R tile rows (m or n index) x 64 k.  TR = operand memory is
// k-major ([K, rows], rows contiguous).
template <int R, int NT, bool TR> struct TileLoader;

template <int R, int NT> struct TileLoader<R, NT, false> {
    static constexpr int NCH = R * 8 / NT;  // 16-byte chunks per thread
    static_assert(NCH >= 1, "tile too small for the block");
    u32x4 regs[NCH];
    __device__ __forceinline__ void gload(const bf16* base, int64_t ld, int row0, int rows, int k0,
                                          int K, int tid) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + i * NT;
            const int r = c >> 3, kc = c & 7;
            const int gr = row0 + r, gk = k0 + kc * 8;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (gr < rows && gk < K) v = *(const u32x4*)(base + (int64_t)gr * ld + gk);
            regs[i] = v;
        }
    }
    __device__ __forceinline__ void sstore(bf16* lds, int tid) const {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + i * NT;
            const int r = c >> 3, kc = c & 7;
            *(u32x4*)(lds + r * 64 + ((kc ^ swz(r)) << 3)) = regs[i];
        }
    }
};

template <int R, int NT> struct TileLoader<R, NT, true> {
    // each thread owns an 8-row x KB-k block: KB 16-byte loads, each 8 rows at one k
    static constexpr int KB = 8 * R / NT;
    static_assert(KB == 2 || KB == 4 || KB == 8, "unsupported tile/block combination");
    static constexpr int NRB = R / 8;
    u32x4 regs[KB];
    __device__ __forceinline__ void gload(const bf16* base, int64_t ld, int row0, int rows, int k0,
                                          int K, int tid) {
        const int rb = tid % NRB, kb = tid / NRB;
        const int gr = row0 + rb * 8;
#pragma unroll
        for (int j = 0; j < KB; ++j) {
            const int gk = k0 + kb * KB + j;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (gr < rows && gk < K) v = *(const u32x4*)(base + (int64_t)gk * ld + gr);
            regs[j] = v;
        }
    }
    __device__ __forceinline__ void sstore(bf16* lds, int tid) const {
        const int rb = tid % NRB, kb = tid / NRB;
        const int ko = kb * KB;  // k offset inside the 64-wide tile
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            // row i of the block: element i of every loaded vector
            uint32_t w[KB / 2];
#pragma unroll
            for (int j = 0; j < KB / 2; ++j) {
                const uint32_t lo = regs[2 * j][i >> 1], hi = regs[2 * j + 1][i >> 1];
                w[j] = (i & 1) ? ((lo >> 16) | (hi & 0xffff0000u)) : ((lo & 0xffffu) | (hi << 16));
            }
            const int r = rb * 8 + i;
            bf16* dst = lds + r * 64 + ((((ko >> 3) ^ swz(r))) << 3) + (ko & 7);
            if constexpr (KB == 8) {
                u32x4 t = {w[0], w[1], w[2], w[3]};
                *(u32x4*)dst = t;
            } else if constexpr (KB == 4) {
                u32x2 t = {w[0], w[1]};
                *(u32x2*)dst = t;
            } else {
                *(uint32_t*)dst = w[0];
            }
        }
    }
};

template <int BM, int BN, int WM, int WN, bool TA, bool TB>
__global__ __launch_bounds__(WM* WN * 64) void gemm_bf16_kernel(const GemmArgs g) {
    constexpr int NT = WM * WN * 64, BK = 64;
    constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32;
    static_assert(TM >= 1 && TN >= 1, "wave tile must hold a 32x32 MFMA tile");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    bf16* As = (bf16*)smem;            // [2][BM*BK]
    bf16* Bs = As + 2 * BM * BK;       // [2][BN*BK]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    int tile_m, tile_n;
    tile_coords(blockIdx.x, g.tiles_m, g.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int b1 = blockIdx.z / g.nb2, b2 = blockIdx.z % g.nb2;
    const bf16* A = (const bf16*)g.A + b1 * g.sA1 + b2 * g.sA2;
    const bf16* B = (const bf16*)g.B + b1 * g.sB1 + b2 * g.sB2;
    const int64_t coff = b1 * g.sC1 + b2 * g.sC2;

    TileLoader<BM, NT, TA> la;
    TileLoader<BN, NT, TB> lb;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int KT = (g.K + BK - 1) / BK;
    la.gload(A, g.lda, m0, g.M, 0, g.K, tid);
    lb.gload(B, g.ldb, n0, g.N, 0, g.K, tid);
    la.sstore(As, tid);
    lb.sstore(Bs, tid);
    __syncthreads();

    const int frow = lane & 31, fk = lane >> 5;
    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        const bool more = kt + 1 < KT;
        if (more) {
            la.gload(A, g.lda, m0, g.M, (kt + 1) * BK, g.K, tid);
            lb.gload(B, g.ldb, n0, g.N, (kt + 1) * BK, g.K, tid);
        }
        const bf16* as = As + cur * BM * BK;
        const bf16* bs = Bs + cur * BN * BK;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            bf16x8 af[TM], bfr[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int r = wm * WTM + i * 32 + frow;
                af[i] = *(const bf16x8*)(as + r * 64 + (((ks * 2 + fk) ^ swz(r)) << 3));
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int r = wn * WTN + j * 32 + frow;
                bfr[j] = *(const bf16x8*)(bs + r * 64 + (((ks * 2 + fk) ^ swz(r)) << 3));
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
        }
        if (more) {
            la.sstore(As + (cur ^ 1) * BM * BK, tid);
            lb.sstore(Bs + (cur ^ 1) * BN * BK, tid);
        }
        __syncthreads();
    }

    // epilogue: lane holds column (lane & 31); register r is row 8*(r/4) + 4*(lane/32) + r%4
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + wn * WTN + j * 32 + (lane & 31);
            if (n >= g.N) continue;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * WTM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (m < g.M) epilogue_elem<bf16>(g, coff, coff, m, n, acc[i][j][r]);
            }
        }
}

// =========================================================================================
// bf16 kernel, DMA generation: tiles go global -> LDS directly (global_load_lds_dwordx4, no
// VGPR staging) through a 4-stage ring of 32-wide k-tiles, MFMA fragments are double-buffered
// in registers so LDS reads of tile t+1 overlap the MFMAs of tile t.
//
// LDS tile formats (one wave-instruction always fills 1024 contiguous bytes, 16 B per lane):
//   KC operand (memory rows are k-contiguous): [rows][32 k], 64 B per row = 4 chunks of 16 B,
//       chunk c of row r at slot c ^ ((r >> 2) & 3); fragments by ds_read_b128.
//   KM operand (memory is k-major, rows contiguous): [32 k][rows], chunk c of k-row k at slot
//       c ^ (4 * (k & 3)); fragments by two ds_read_b64_tr_b16 (the hardware transposes a
//       4k x 16row block across 16 lanes: lane j reads row k0 + j/4, cols 4*(j%4)..+3 and
//       receives column j, k0..k0+3).
// Rows beyond M / N are clamped to the last valid row (their results are never stored);
// K must be a multiple of 32.
// =========================================================================================
typedef __attribute__((address_space(3))) void lds_ptr_t;
typedef const __attribute__((address_space(1))) void gbl_ptr_t;
typedef __attribute__((ext_vector_type(4))) short s16x4;

// Ask the machine scheduler for "one MFMA, then its share of NMEM memory instructions" NMFMA times:
// the memory instructions of a region (LDS fragment reads or DMA issues) are spread between the
// MFMAs instead of being bunched in front of a full wait.
template <int NMFMA, int NMEM, int MEM_MASK> __device__ __forceinline__ void interleave_mfma_with() {
    static_for(
        [&](auto idx) {
            constexpr int i = decltype(idx)::value;
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            constexpr int n = (NMEM * (i + 1)) / NMFMA - (NMEM * i) / NMFMA;
            if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(MEM_MASK, n, 0);
        },
        std::make_integer_sequence<int, NMFMA>{});
}

template <int N> __device__ __forceinline__ void wait_vmcnt_lgkm0() {
    // s_waitcnt vmcnt(N) lgkmcnt(0): vmcnt[3:0] | expcnt(7) << 4 | lgkmcnt << 8 | vmcnt[5:4] << 14
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (0 << 8) | ((N >> 4) << 14));
}

// One wave-wide 16-byte-per-lane global -> LDS transfer (global_load_lds_dwordx4; the LDS target
// is M0 + lane * 16).  Issued as inline assembly on purpose: while the compiler sees such a load in
// flight it turns EVERY wait for an LDS read into lgkmcnt(0), i.e. each fragment wait would drain
// all outstanding fragment reads.  Unseen, the fragment waits keep their exact counts.  The price:
// the compiler does not count these loads in vmcnt either - the main loop waits for them explicitly
// (it always did), and nothing else may touch the target stage or leave the kernel's main loop
// without an explicit vmcnt wait.
__device__ __forceinline__ void dma16(const void* src, const unsigned char* lds_dst) {
    const unsigned m0 = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)(lds_ptr_t*)lds_dst);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(m0), "v"(src) : "m0");
}

// 3x3 convolution (stride 1, pad 1, NHWC) as an implicit GEMM: the patch matrix [pixels, 9 * channels] is never
// built, the A loader gathers its rows from the activation tensor instead.
struct ConvArgs {
    int h, w, c;      // image height / width, channels of the gathered tensor (a multiple of the 64-wide k-tile)
    int b_every;      // input-gradient mode: k-tiles per tap of the B operand ...
    int64_t b_wrap;   // ... and what its pointers move by (on top of the k-tile step) when the tap changes
};
// what the taps outside the image read
__device__ __attribute__((aligned(128))) unsigned char bb_zero_line[128];

// VIS: issue through the compiler builtin instead (the compiler then sees the load and waits lgkmcnt(0)
// for every fragment read, which keeps the waves of a block in lock step)
// CONV 1 (row-contiguous operand, 64-wide k-tiles): row p of the operand is pixel p's 3x3 neighbourhood,
// k = tap * channels + channel; a k-tile lies inside one tap, so each lane reads 16 bytes of the neighbouring
// pixel's channel vector, or of a line of zeros where the tap falls outside the image.
// CONV 2 (k-major operand): the weight [out, 9, in] read as B[k = (8 - tap) * out + o, n = i] (the flipped
// filter of the input gradient): rows o advance by the k-tile, and every out / 64 k-tiles the tap changes.
template <int BR, bool KM, int NW, int BK = 32, bool VIS = false, int CONV = 0> struct DmaOperand {
    static constexpr int BYTES = BR * BK * 2;
    static constexpr int ROUNDS = BYTES / (1024 * NW);  // instructions per thread per k-tile
    static_assert(ROUNDS >= 1, "tile too small for the block");
    static_assert(CONV == 0 || (CONV == 1 && !KM && BK == 64) || ((CONV == 2 || CONV == 3) && KM), "convolution loaders: see above");
    const bf16* src[ROUNDS];
    int64_t step;  // elements to advance per k-tile
    // CONV 1: per round the taps that lie inside the image (bit t = tap t), then wave-uniform position in K
    unsigned inside[ROUNDS];
    const bf16* zero;
    int tap, c0, kstep, cw, cc;
    int64_t tapoff;
    // CONV 2
    int cnt, every;
    int64_t wrap;
    // CONV 3: image coordinates of the pixel each round reads next, the block's tap, the k-tile step in pixels
    int py[ROUNDS], px[ROUNDS];
    int tdy, tdx, dpy, dpx, ch;

    __device__ __forceinline__ void init(const bf16* base, int64_t ld, int row0, int rows, int tid) {
        const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
        for (int i = 0; i < ROUNDS; ++i) {
            const int q = i * NW + wave;
            if constexpr (!KM && BK == 64) {
                // 64-wide k-tiles: one instruction takes 8 rows x 128 B, whole cache lines
                const int r = q * 8 + (lane >> 3);
                const int c = (lane & 7) ^ ((r >> 1) & 7);
                const int gr = min(row0 + r, rows - 1);
                src[i] = base + (int64_t)gr * ld + c * 8;
            } else if constexpr (!KM) {
                const int r = q * 16 + (lane >> 2);
                const int c = (lane & 3) ^ ((r >> 2) & 3);
                const int gr = min(row0 + r, rows - 1);
                src[i] = base + (int64_t)gr * ld + c * 8;
            } else {
                constexpr int CPR = BR / 8, RPI = 64 / CPR;
                const int k = q * RPI + lane / CPR;
                const int c = (lane % CPR) ^ (4 * (k & 3));
                const int gc = min(row0 + c * 8, rows - 8);
                src[i] = base + (int64_t)k * ld + gc;
            }
        }
        step = KM ? BK * ld : BK;
    }
    // CONV 1: base = the activation tensor [pixels, cv.c]; src[i] points at the lane's chunk of the centre pixel
    __device__ __forceinline__ void init_conv(const bf16* base, int row0, int rows, int tid, const ConvArgs& cv) {
        const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
        for (int i = 0; i < ROUNDS; ++i) {
            const int q = i * NW + wave;
            const int r = q * 8 + (lane >> 3);
            const int c = (lane & 7) ^ ((r >> 1) & 7);
            const int gr = min(row0 + r, rows - 1);
            const int pix = gr % (cv.h * cv.w), py = pix / cv.w, px = pix % cv.w;
            unsigned m = 0;
#pragma unroll
            for (int t = 0; t < 9; ++t) {
                const int sy = py + t / 3 - 1, sx = px + t % 3 - 1;
                if (sy >= 0 && sy < cv.h && sx >= 0 && sx < cv.w) m |= 1u << t;
            }
            inside[i] = m;
            src[i] = base + (int64_t)gr * cv.c + c * 8;
        }
        zero = (const bf16*)(bb_zero_line + (lane & 7) * 16);
        step = 0;
        tap = 0; c0 = 0; kstep = BK; cw = cv.w; cc = cv.c;
        tapoff = (int64_t)(-cv.w - 1) * cv.c;
    }
    // CONV 2: after init() with base already at tap 8 of the weight
    __device__ __forceinline__ void init_wrap(const ConvArgs& cv) {
        cnt = 0; every = cv.b_every; wrap = cv.b_wrap;
    }
    // CONV 3 (k-major operand): the patch matrix [pixels, 9 * c] of the tensor at base as the B operand of a
    // weight gradient.  A column tile (col0 .. col0 + BR - 1, inside one tap since c % BR == 0) reads channels
    // of the pixel `tap` away from pixel k: rows advance by the k-tile, the lane's image coordinates with them.
    __device__ __forceinline__ void init_conv_km(const bf16* base, int col0, int tid, int h, int w, int c, int pix0) {
        const int lane = tid & 63, wave = tid >> 6;
        const int t = col0 / c, ci0 = col0 - t * c;
        tdy = t / 3 - 1; tdx = t % 3 - 1; ch = h; cw = w;
        dpy = BK / w; dpx = BK % w;
#pragma unroll
        for (int i = 0; i < ROUNDS; ++i) {
            const int q = i * NW + wave;
            constexpr int CPR = BR / 8, RPI = 64 / CPR;
            const int k = q * RPI + lane / CPR;
            const int cch = (lane % CPR) ^ (4 * (k & 3));
            const int p = pix0 + k, pix = p % (h * w);
            py[i] = pix / w;
            px[i] = pix - py[i] * w;
            src[i] = base + ((int64_t)p + tdy * w + tdx) * c + ci0 + cch * 8;
        }
        zero = (const bf16*)(bb_zero_line + (lane & 7) * 16);
        step = (int64_t)BK * c;
    }
    // past the end of K: the last tile is fetched again and again
    __device__ __forceinline__ void stop() {
        step = 0;
        if constexpr (CONV == 1) kstep = 0;
        if constexpr (CONV == 2) wrap = 0;
        if constexpr (CONV == 3) dpy = dpx = 0;
    }
    __device__ __forceinline__ const bf16* source(int i) const {
        if constexpr (CONV == 1) return ((inside[i] >> tap) & 1u) ? src[i] + (tapoff + c0) : zero;
        else if constexpr (CONV == 3)
            return ((unsigned)(py[i] + tdy) < (unsigned)ch && (unsigned)(px[i] + tdx) < (unsigned)cw) ? src[i] : zero;
        else return src[i];
    }
    // CONV 3: round i moves on by one k-tile of pixels (BK / w + 1 <= h: at most one image boundary per step)
    __device__ __forceinline__ void next_pixels(int i) {
        if constexpr (CONV == 3) {
            px[i] += dpx;
            py[i] += dpy;
            if (px[i] >= cw) {
                px[i] -= cw;
                ++py[i];
            }
            if (py[i] >= ch) py[i] -= ch;
        }
    }
    // after the last instruction of a k-tile
    __device__ __forceinline__ void advance() {
        if constexpr (CONV == 1) {
            c0 += kstep;
            if (c0 >= cc) {
                c0 = 0;
                ++tap;
                tapoff = (int64_t)((tap / 3 - 1) * cw + (tap % 3 - 1)) * cc;
            }
        } else if constexpr (CONV == 2) {
            if (++cnt == every) {
                cnt = 0;
#pragma unroll
                for (int i = 0; i < ROUNDS; ++i) src[i] += wrap;
            }
        }
    }
    __device__ __forceinline__ void issue(unsigned char* tile, int wave) {
#pragma unroll
        for (int i = 0; i < ROUNDS; ++i) {
            if constexpr (VIS) __builtin_amdgcn_global_load_lds((gbl_ptr_t*)source(i), (lds_ptr_t*)(tile + (i * NW + wave) * 1024), 16, 0, 0);
            else dma16(source(i), tile + (i * NW + wave) * 1024);
            src[i] += step;
            next_pixels(i);
        }
        advance();
    }
    template <int I> __device__ __forceinline__ void issue_one(unsigned char* tile, int wave) {
        dma16(source(I), tile + (I * NW + wave) * 1024);
        src[I] += step;
        next_pixels(I);
        if constexpr (I == ROUNDS - 1) advance();
    }
};

// per-lane fragment offsets (bytes inside an operand tile) and the fragment fetch
template <int BR, int T, bool KM, int BK = 32> struct FragReader {
    int off[KM ? T : 1];
    int sw, hi;
    __device__ __forceinline__ void init(int wbase, int lane) {
        hi = lane >> 5;
        if constexpr (!KM) {
            sw = BK == 64 ? ((lane & 31) >> 1) & 7 : ((lane & 31) >> 2) & 3;
            off[0] = (wbase + (lane & 31)) * (BK * 2);
        } else {
            const int j4 = (lane & 15) >> 2;
            const int lo = ((lane >> 4) & 1) * 2 + ((lane & 3) >> 1);
            const int within = (lane & 1) * 4;  // element offset inside the 16-byte chunk
            sw = 0;
#pragma unroll
            for (int t = 0; t < T; ++t) {
                const int c4 = ((wbase >> 5) + t) ^ j4;  // chunk-of-four index after the swizzle
                off[t] = (hi * 8 + j4) * (BR * 2) + ((c4 * 4 + lo) << 4) + within * 2;
            }
        }
    }
    __device__ __forceinline__ bf16x8 load(const unsigned char* tile, int t, int ks) const {
        if constexpr (!KM) {
            return *(const bf16x8*)(tile + off[0] + t * (32 * BK * 2) + (((ks * 2 + hi) ^ sw) << 4));
        } else {
            const unsigned char* p = tile + off[t] + ks * 16 * (BR * 2);
            s16x4 lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(p));
            s16x4 hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(p + 4 * (BR * 2)));
            typedef __attribute__((ext_vector_type(8))) short s16x8;
            s16x8 v = __builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7);
            return __builtin_bit_cast(bf16x8, v);
        }
    }
};

// STATS 1: the epilogue also leaves the column statistics of the stored (bf16-rounded) output per 32-row strip, for the
// batch normalisation that follows a convolution (its statistics pass then has nothing left to read).
// STATS 2: the product is the gradient that arrives at a batch normalisation (+ ReLU, applied by the epilogue kind);
// the epilogue also leaves that normalisation's backward sums per strip (BnBwdArgs), so that its backward pass has no
// reduction over the tensor left.
template <int BM, int BN, int WM, int WN, bool AKM, bool BKM, bool DB, int STAGES, int BK = 32, bool VIS = false, int CONV = 0,
          int STATS = 0, bool DROP = false>
__device__ __forceinline__ void gemm_bf16_dma_body(const GemmArgs& g, const int block_id, const int batch_id,
                                                   const bool logical_id = false, const ConvArgs& cv = ConvArgs{},
                                                   const BnBwdArgs& bn = BnBwdArgs{}) {
    constexpr int NW = WM * WN;
    static_assert(BK == 64 ? (STAGES >= 2 && DB) : STAGES >= 3,
                  "32-wide k-tiles: the ring needs one stage being read, one landing, one in flight; "
                  "64-wide k-tiles alternate between two stages or rotate through more");
    constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32;
    // CONV 1: forward 3x3 convolution (A gathered); CONV 2: its input gradient (A gathered, B the flipped filter)
    // CONV 3: its weight gradient (B = the patch matrix, gathered)
    static_assert(CONV == 0 || (CONV == 3 ? AKM && BKM : !AKM && (CONV == 2) == BKM),
                  "implicit convolution: NT forward, NN input gradient, TN weight gradient");
    using OpA = DmaOperand<BM, AKM, NW, BK, VIS, CONV == 1 || CONV == 2 ? 1 : 0>;
    using OpB = DmaOperand<BN, BKM, NW, BK, VIS, CONV >= 2 ? CONV : 0>;
    constexpr int STAGE_BYTES = OpA::BYTES + OpB::BYTES;
    constexpr int LOADS = OpA::ROUNDS + OpB::ROUNDS;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    int tile_m, tile_n;
    // the 32 tiles an XCD holds at a time read BM * rows + BN * columns operand rows: 4 x 8 tiles of 256 x 128 read
    // 2048, 8 x 4 read 2560
    constexpr int GROUP_M = (BM == 256 && BN == 128 && CONV == 0) ? 4 : 8;
    if (logical_id) panel_coords<8>(block_id, g.tiles_m, g.tiles_n, tile_m, tile_n);
    else tile_coords<GROUP_M>(block_id, g.tiles_m, g.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int b1 = batch_id / g.nb2, b2 = batch_id % g.nb2;
    const bf16* A = (const bf16*)g.A + b1 * g.sA1 + b2 * g.sA2;
    const bf16* B = (const bf16*)g.B + b1 * g.sB1 + b2 * g.sB2;
    const int64_t coff = b1 * g.sC1 + b2 * g.sC2;

    OpA opa;
    OpB opb;
    if constexpr (CONV == 1 || CONV == 2) opa.init_conv(A, m0, g.M, tid, cv);
    else opa.init(A, g.lda, m0, g.M, tid);
    if constexpr (CONV == 3) opb.init_conv_km(B, n0, tid, g.conv_h, g.conv_w, g.conv_c, g.conv_row0);
    else opb.init(B, g.ldb, n0, g.N, tid);
    if constexpr (CONV == 2) opb.init_wrap(cv);
    FragReader<BM, TM, AKM, BK> fa;
    FragReader<BN, TN, BKM, BK> fb;
    fa.init(wm * WTM, lane);
    fb.init(wn * WTN, lane);

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    struct Frags {
        bf16x8 a[2][TM], b[2][TN];
    };
    Frags f0, f1;
    const int KT = g.K / BK;

    // ring positions: tile t lives in stage t % STAGES
    int issue_stage = 0, read_stage = 0;
    auto issue_tile = [&]() {
        unsigned char* st = smem + issue_stage * STAGE_BYTES;
        opa.issue(st, wave);
        opb.issue(st + OpA::BYTES, wave);
        issue_stage = issue_stage + 1 == STAGES ? 0 : issue_stage + 1;
    };
    auto load_frags = [&](Frags& f) {
        const unsigned char* st = smem + read_stage * STAGE_BYTES;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int i = 0; i < TM; ++i) f.a[ks][i] = fa.load(st, i, ks);
#pragma unroll
            for (int j = 0; j < TN; ++j) f.b[ks][j] = fb.load(st + OpA::BYTES, j, ks);
        }
        read_stage = read_stage + 1 == STAGES ? 0 : read_stage + 1;
    };
    // bias gradient riding along: the waves of the first block column (and first wave column)
    // add up the A fragments they hold anyway: lane (m, kg) sees 8 of the 16 k values per step
    const bool do_colsum = AKM && g.colsum != nullptr && tile_n == 0 && wn == 0;
    float csum[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) csum[i] = 0.f;
    auto mfma_step = [&](const Frags& f, int ks) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.a[ks][i], f.b[ks][j], acc[i][j], 0, 0, 0);
        if constexpr (AKM) {
            if (do_colsum) {
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    float t = 0.f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) t += (float)f.a[ks][i][e];
                    csum[i] += t;
                }
            }
        }
    };
    // One quarter / half of a tile placed by hand: MFMA m of step ks, then its share of ND DMA
    // instructions into stage `dst` and of the fragment reads of (stage `src`, half h) into `nf` (the
    // reads ride on the first FM MFMAs so that the last ones cover their latency), each group fenced:
    // the DMA instructions are inline assembly, opaque to the scheduler's group hints, and unfenced
    // they end up bunched behind the barrier.
    // (KOFF: the step issues DMA instructions KOFF .. KOFF + ND - 1 of the k-tile)
    auto placed_step = [&](const Frags& f, auto ks_c, auto nd_c, unsigned char* dst, auto reads_c, Frags& nf,
                           const unsigned char* src, int h, auto koff_c) {
        constexpr int ks = decltype(ks_c)::value, ND = decltype(nd_c)::value, KOFF = decltype(koff_c)::value;
        constexpr bool READS = decltype(reads_c)::value;
        constexpr int NM = TM * TN, NF = 2 * (TM + TN), FM = NM > 2 ? NM - 2 : NM;
        static_for(
            [&](auto idx) {
                constexpr int m = decltype(idx)::value, i = m / TN, j = m % TN;
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.a[ks][i], f.b[ks][j], acc[i][j], 0, 0, 0);
                if constexpr (AKM && j == 0) {
                    if (do_colsum) {
                        float t = 0.f;
#pragma unroll
                        for (int e = 0; e < 8; ++e) t += (float)f.a[ks][i][e];
                        csum[i] += t;
                    }
                }
                static_for(
                    [&](auto d) {
                        constexpr int k = KOFF + (ND * m) / NM + decltype(d)::value;
                        if constexpr (k < OpA::ROUNDS) opa.template issue_one<k>(dst, wave);
                        else opb.template issue_one<k - OpA::ROUNDS>(dst + OpA::BYTES, wave);
                    },
                    std::make_integer_sequence<int, (ND * (m + 1)) / NM - (ND * m) / NM>{});
                if constexpr (READS && m < FM) {
                    static_for(
                        [&](auto r) {
                            constexpr int q = (NF * m) / FM + decltype(r)::value, fk = q / (TM + TN), t = q % (TM + TN);
                            if constexpr (t < TM) nf.a[fk][t] = fa.load(src, t, h * 2 + fk);
                            else nf.b[fk][t - TM] = fb.load(src + OpA::BYTES, t - TM, h * 2 + fk);
                        },
                        std::make_integer_sequence<int, (NF * (m + 1)) / FM - (NF * m) / FM>{});
                }
                __builtin_amdgcn_sched_barrier(0);
            },
            std::make_integer_sequence<int, NM>{});
    };
    // Steady state is branch-free: a tile is issued every iteration (past the end of K the
    // sources stop advancing, so the last tile is fetched again into a stage nobody reads),
    // hence exactly STAGES-2 newer tiles are in flight whenever a wave waits for the next tile.
    auto sync_tile = [&]() {
        asm volatile("" ::: "memory");
        wait_vmcnt_lgkm0<(STAGES - 2) * LOADS>();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    auto stop_at_end = [&](int next_tile) {
        if (next_tile >= KT) {
            opa.stop();
            opb.stop();
        }
    };

    // the operand of the epilogue kinds that read one, fetched a patch ahead of its use: the four 16-byte pieces of
    // patch q; patch 0's go out at the top of the last k-tile
    constexpr int PLD = 68;
    constexpr int NP = (TN + 1) / 2;   // pairs per row of accumulator tiles, the last one possibly a single
    const int prow = lane >> 3, pcol = (lane & 7) * 8;
    // Only on the large tiles (one block per CU, two waves per SIMD whatever the kernel's register count): on the
    // small ones the 32 registers would cost a resident block.
    // Some of the other kernels fetch a patch's operand(s) in one go at the top of that patch: the pointers of GemmArgs
    // may alias as far as the compiler knows, so left inside the row loop every load waits behind the previous row's
    // store (four round trips in a row per patch instead of one).
    // (HOIST: where that does not cost a resident block -- the kernels with the BatchNorm backward sums, whose three
    // operand reads per row are most of their epilogue)
    constexpr bool PREF = BM * BN >= 256 * 128 && !VIS && CONV == 0 && STATS == 0;
    constexpr bool HOIST = STATS == 2;
    const bf16* opnd = PREF || HOIST ? epilogue_operand(g) : nullptr;
    u32x4 opc[PREF || HOIST ? 4 : 1], opn[PREF ? 4 : 1];
    u32x4 xw[STATS == 2 ? 4 : 1], rw[STATS == 2 ? 4 : 1];   // STATS 2: the normalisation's input and the skip gradient
    auto fetch = [&](auto q_c, u32x4 (&dst)[PREF || HOIST ? 4 : 1]) {
        if constexpr (!(PREF || HOIST)) return;
        constexpr int q = decltype(q_c)::value, i = q / NP, jp = q % NP;
        constexpr int NH = (jp * 2 + 1 < TN) ? 2 : 1;
        const int n = n0 + wn * WTN + jp * 64 + pcol;
        const bool live = (NH == 2 || pcol < 32) && n < g.N;
        const int m_first = m0 + wm * WTM + i * 32 + prow;
#pragma unroll
        for (int it = 0; it < (PREF || HOIST ? 4 : 1); ++it) {
            const int m = m_first + it * 8;
            dst[it] = u32x4{0u, 0u, 0u, 0u};
            if (opnd && live && m < g.M) dst[it] = *(const u32x4*)(opnd + coff + (int64_t)m * g.ldaux + n);
            if constexpr (STATS == 2) {
                xw[it] = rw[it] = u32x4{0u, 0u, 0u, 0u};
                if (live && m < g.M) {
                    xw[it] = *(const u32x4*)((const bf16*)bn.x + coff + (int64_t)m * g.ldc + n);
                    if (g.epilogue == BB_EPI_MUL_POS && g.resid) rw[it] = *(const u32x4*)((const bf16*)g.resid + coff + (int64_t)m * g.ldaux + n);
                }
            }
        }
    };

    if constexpr (BK == 64) {
        // Two stages of 64-wide k-tiles, each multiplied as two 32-wide halves from the two fragment
        // sets.  Per tile one barrier, in the middle of its second half: by then every wave has read
        // the tile's last fragments (so its stage can take tile kt+2) and tile kt+1, issued one whole
        // tile earlier, has to have landed (its first fragments are read right after).
        auto load_half = [&](Frags& f, const unsigned char* st, int h) {
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
                for (int i = 0; i < TM; ++i) f.a[ks][i] = fa.load(st, i, h * 2 + ks);
#pragma unroll
                for (int j = 0; j < TN; ++j) f.b[ks][j] = fb.load(st + OpA::BYTES, j, h * 2 + ks);
            }
        };
        constexpr int FRAG_READS = 2 * (TM * (AKM ? 2 : 1) + TN * (BKM ? 2 : 1));
        // prologue: tiles 0 and 1 with two stages, 0..STAGES-2 with more (tile kt+STAGES-1 then goes out
        // at the top of iteration kt, into the stage tile kt-1 has left)
        constexpr int PRO = STAGES == 2 ? 2 : STAGES - 1;
#pragma unroll
        for (int t = 0; t < PRO; ++t) {
            stop_at_end(t + 1);
            issue_tile();
        }
        asm volatile("" ::: "memory");
        wait_vmcnt_lgkm0<(PRO - 1) * LOADS>();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        load_half(f0, smem, 0);
        int rs = 0;
        for (int kt = 0; kt < KT; ++kt) {
            const unsigned char* cur = smem + rs * STAGE_BYTES;
            rs = rs + 1 == STAGES ? 0 : rs + 1;
            const unsigned char* nxt = smem + rs * STAGE_BYTES;
            if constexpr (STAGES >= 3) {
                if constexpr (PREF) {
                    if (kt == KT - 1) fetch(std::integral_constant<int, 0>{}, opc);
                }
                // the DMA instructions of tile kt+STAGES-1 a third each between the MFMAs of the first three quarters
                // (issued in one burst at the top they queue up in front of the texture path and the waves behind
                // them: 2-5 % slower), the second half's fragment reads between the first MFMAs
                stop_at_end(kt + STAGES);
                unsigned char* into = smem + issue_stage * STAGE_BYTES;
                issue_stage = issue_stage + 1 == STAGES ? 0 : issue_stage + 1;
                constexpr int THIRD = LOADS / 3;
                placed_step(f0, std::integral_constant<int, 0>{}, std::integral_constant<int, THIRD>{}, into, std::true_type{}, f1,
                            cur, 1, std::integral_constant<int, 0>{});
                placed_step(f0, std::integral_constant<int, 1>{}, std::integral_constant<int, THIRD>{}, into, std::false_type{}, f1,
                            cur, 1, std::integral_constant<int, THIRD>{});
                placed_step(f1, std::integral_constant<int, 0>{}, std::integral_constant<int, LOADS - 2 * THIRD>{}, into,
                            std::false_type{}, f1, cur, 1, std::integral_constant<int, 2 * THIRD>{});
            } else {
                load_half(f1, cur, 1);
                mfma_step(f0, 0);
                mfma_step(f0, 1);
                interleave_mfma_with<2 * TM * TN, FRAG_READS, 0x100>();
                mfma_step(f1, 0);
            }
            // scheduling fences: without them the compiler sinks this third quarter below the barrier
            // and bunches the next tile's fragment reads at the end of the iteration, right in front
            // of the wait for them
            __builtin_amdgcn_sched_barrier(0);
            asm volatile("" ::: "memory");
            wait_vmcnt_lgkm0<(STAGES - 2) * LOADS>();
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            // last quarter: the DMA instructions of tile kt+2 (two stages: into the stage of tile kt)
            // and the first fragment reads of tile kt+1 between its MFMAs
            unsigned char* dst = smem + issue_stage * STAGE_BYTES;
            if constexpr (STAGES == 2) {
                stop_at_end(kt + 3);
                issue_stage = issue_stage + 1 == STAGES ? 0 : issue_stage + 1;
            }
            placed_step(f1, std::integral_constant<int, 1>{}, std::integral_constant<int, STAGES == 2 ? LOADS : 0>{}, dst,
                        std::true_type{}, f0, nxt, 0, std::integral_constant<int, 0>{});
            __builtin_amdgcn_sched_barrier(0);
        }
    } else {
    // prologue: tiles 0..STAGES-2 (clamped to the last tile when K is short)
#pragma unroll
    for (int t = 0; t < STAGES - 1; ++t) {
        stop_at_end(t + 1);
        issue_tile();
    }
    sync_tile();
    if constexpr (DB) {
        // fragments of tile kt+1 are fetched while the second half of tile kt is multiplied,
        // into the other register set
        // Hand placement pays on the 256x256 tile (eight MFMAs per half to place things between: +1..5 %);
        // on the smaller tiles and with two k-major operands (twice the fragment read instructions) the
        // scheduler's own order is as good or better.
        constexpr bool PLACED = BM == 256 && BN == 256 && !AKM;
        auto body = [&](int kt, Frags& cur, Frags& nxt) {
          if constexpr (PLACED) {
            // first half: the DMA instructions of tile kt+STAGES-1 between its MFMAs; second half, behind
            // the barrier: the fragment reads of tile kt+1
            stop_at_end(kt + STAGES);
            unsigned char* dst = smem + issue_stage * STAGE_BYTES;
            issue_stage = issue_stage + 1 == STAGES ? 0 : issue_stage + 1;
            placed_step(cur, std::integral_constant<int, 0>{}, std::integral_constant<int, LOADS>{}, dst, std::false_type{},
                        nxt, smem, 0, std::integral_constant<int, 0>{});
            sync_tile();
            const unsigned char* st = smem + read_stage * STAGE_BYTES;
            read_stage = read_stage + 1 == STAGES ? 0 : read_stage + 1;
            placed_step(cur, std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{}, dst, std::true_type{}, nxt,
                        st, 0, std::integral_constant<int, 0>{});
          } else {
            constexpr int FRAG_READS = 2 * (TM * (AKM ? 2 : 1) + TN * (BKM ? 2 : 1));
            stop_at_end(kt + STAGES);
            issue_tile();
            mfma_step(cur, 0);
            interleave_mfma_with<TM * TN, LOADS, 0x020>();   // DMA issues between the first-half MFMAs
            sync_tile();
            load_frags(nxt);
            mfma_step(cur, 1);
            interleave_mfma_with<TM * TN, FRAG_READS, 0x100>();  // next tile's fragment reads between the rest
          }
        };
        load_frags(f0);
        int kt = 0;
        for (; kt + 1 < KT; kt += 2) {
            body(kt, f0, f1);
            body(kt + 1, f1, f0);
        }
        if (kt < KT) body(kt, f0, f1);
    } else {
        // single fragment set: other resident waves cover LDS latency and barrier waits
        for (int kt = 0; kt < KT; ++kt) {
            stop_at_end(kt + STAGES);
            issue_tile();
            load_frags(f0);
            mfma_step(f0, 0);
            mfma_step(f0, 1);
            sync_tile();
        }
    }
    }

    if constexpr (AKM) {
        if (do_colsum) {
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const float t = csum[i] + __shfl_xor(csum[i], 32, 64);
                const int m = m0 + wm * WTM + i * 32 + (lane & 31);
                if (lane < 32 && m < g.M) g.colsum[m] += t;
            }
        }
    }

    // Epilogue through LDS: every wave parks two horizontally adjacent 32x32 accumulator tiles in a
    // private [32][64 (+4 pad)] fp32 patch; then one wave instruction covers 8 rows x 64 columns, lane l
    // taking 8 consecutive columns of row l/8, so every global load / store of the epilogue moves whole
    // 128-byte row segments (256 bytes for fp32 outputs).
    // An odd tile count per row ends with a single tile: its 32 columns use half of the patch and half of
    // the lanes of the row pass.
    if constexpr (PREF && !(BK == 64 && STAGES >= 3)) fetch(std::integral_constant<int, 0>{}, opc);
    wait_vmcnt_lgkm0<0>();  // the tiles issued past the end of K have to land before their stages become the patch
    __syncthreads();
    float* patch = (float*)smem + wave * (32 * PLD);
    static_for(
        [&](auto idx) {
            constexpr int i = decltype(idx)::value / NP, jp = decltype(idx)::value % NP;
            constexpr int NH = (jp * 2 + 1 < TN) ? 2 : 1;
#pragma unroll
            for (int h = 0; h < NH; ++h)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    patch[(8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * PLD + h * 32 + (lane & 31)] = acc[i][jp * 2 + h][r] * g.alpha;
            asm volatile("" ::: "memory");
            if constexpr (HOIST) fetch(idx, opc);
            else if constexpr (decltype(idx)::value + 1 < TM * NP) fetch(std::integral_constant<int, decltype(idx)::value + 1>{}, opn);
            const int n = n0 + wn * WTN + jp * 64 + pcol;
            const bool live = (NH == 2 || pcol < 32) && n < g.N;
            // per patch: the bias of the lane's eight columns once, the offsets of its first row by multiplication
            // and of the other three by addition (a 64-bit multiply is several quarter-rate instructions)
            float b8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            if (g.bias && live) load_vec((const bf16*)g.bias + n, b8);
            const int m_first = m0 + wm * WTM + i * 32 + prow;
            int64_t ci = coff + (int64_t)m_first * g.ldc + n, xi = coff + (int64_t)m_first * g.ldaux + n;
            // STATS 2: the lane's sums over its four rows, for its eight columns
            float mu8[8], rs8[8], sg[8], sgx[8];
            if constexpr (STATS == 2) {
#pragma unroll
                for (int e = 0; e < 8; ++e) mu8[e] = rs8[e] = sg[e] = sgx[e] = 0.f;
                if (live) {
                    const f32x4 m_lo = *(const f32x4*)(bn.mean + n), m_hi = *(const f32x4*)(bn.mean + n + 4);
                    const f32x4 r_lo = *(const f32x4*)(bn.rstd + n), r_hi = *(const f32x4*)(bn.rstd + n + 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        mu8[e] = m_lo[e];
                        mu8[4 + e] = m_hi[e];
                        rs8[e] = r_lo[e];
                        rs8[4 + e] = r_hi[e];
                    }
                }
            }
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const int m = m_first + it * 8;
                float v[8];
                const f32x4 lo = *(const f32x4*)(patch + (it * 8 + prow) * PLD + pcol);
                const f32x4 hi = *(const f32x4*)(patch + (it * 8 + prow) * PLD + pcol + 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = lo[e];
                    v[4 + e] = hi[e];
                }
                if (live && m < g.M) {
                    epilogue_vec8_at<DROP, PREF || HOIST, HOIST>(g, ci, xi, m, n, v, b8, opc[PREF || HOIST ? it : 0], rw[HOIST ? it : 0]);
                    if constexpr (STATS == 2) {
                        float xv[8];
                        unpack_bf16x8(xw[it], xv);
#pragma unroll
                        for (int e = 0; e < 8; ++e) bn_bwd_sums_add(bf2f(f2bf(v[e])) /* what was stored */, xv[e], mu8[e], rs8[e], sg[e], sgx[e]);
                    }
                }
                ci += 8 * (int64_t)g.ldc;
                xi += 8 * (int64_t)g.ldaux;
            }
            if constexpr (STATS == 2) {
                // the eight row groups' sums through the patch (all of it has been read): rows 0..7 sum g, rows 8..15
                // sum g xhat, then lane = column adds the eight up in row order
                asm volatile("" ::: "memory");
                *(f32x4*)(patch + prow * PLD + pcol) = f32x4{sg[0], sg[1], sg[2], sg[3]};
                *(f32x4*)(patch + prow * PLD + pcol + 4) = f32x4{sg[4], sg[5], sg[6], sg[7]};
                *(f32x4*)(patch + (8 + prow) * PLD + pcol) = f32x4{sgx[0], sgx[1], sgx[2], sgx[3]};
                *(f32x4*)(patch + (8 + prow) * PLD + pcol + 4) = f32x4{sgx[4], sgx[5], sgx[6], sgx[7]};
                asm volatile("" ::: "memory");
                float t0 = 0.f, t1 = 0.f;
#pragma unroll
                for (int r = 0; r < 8; ++r) {
                    t0 = __fadd_rn(t0, patch[r * PLD + lane]);
                    t1 = __fadd_rn(t1, patch[(8 + r) * PLD + lane]);
                }
                const int strip_row = m0 + wm * WTM + i * 32;
                const int nc = n0 + wn * WTN + jp * 64 + lane;
                if (strip_row < g.M && nc < g.N && (NH == 2 || lane < 32)) {
                    float* o = bn.strips + ((int64_t)(strip_row >> 5) * 2) * g.N + nc;
                    o[0] = t0;
                    o[g.N] = t1;
                }
            }
            if constexpr (STATS == 1) {
                // Column statistics of this 32-row strip straight from the patch: lane = column, 32 conflict-free LDS
                // reads.  The patch holds what is stored (alpha = 1, no bias, no epilogue), rounded here as the
                // store rounds it; the pivot is the strip's first row.
                const int strip_row = m0 + wm * WTM + i * 32, nrows = min(32, g.M - strip_row);
                const int nc = n0 + wn * WTN + jp * 64 + lane;
                const float piv = bf2f(f2bf(patch[lane]));
                float s1 = 0.f, s2 = 0.f;
#pragma unroll
                for (int r = 0; r < 32; ++r) {
                    const float dv = bf2f(f2bf(patch[r * PLD + lane])) - piv;
                    if (r < nrows) {
                        s1 += dv;
                        s2 += dv * dv;
                    }
                }
                if (g.strip_stats && nrows > 0 && nc < g.N && (NH == 2 || lane < 32)) {
                    float* o = g.strip_stats + ((int64_t)(strip_row >> 5) * 3) * g.N + nc;
                    o[0] = piv;
                    o[g.N] = s1;
                    o[2 * (int64_t)g.N] = s2;
                }
            }
            asm volatile("" ::: "memory");
            if constexpr (PREF) {
#pragma unroll
                for (int it = 0; it < 4; ++it) opc[it] = opn[it];
            }
        },
        std::make_integer_sequence<int, TM * NP>{});
}

// DROP: the epilogue can apply dropout (g.drop).  A kernel of its own, so that the keep decisions' registers cost the
// kernels without dropout nothing (they decide how many blocks of the small tiles a CU holds).
template <int BM, int BN, int WM, int WN, bool AKM, bool BKM, bool DB, int STAGES, int BK, bool DROP = false>
__global__ __launch_bounds__(WM* WN * 64) void gemm_bf16_dma_kernel(const GemmArgs g) {
    gemm_bf16_dma_body<BM, BN, WM, WN, AKM, BKM, DB, STAGES, BK, false, 0, 0, DROP>(g, blockIdx.x, blockIdx.z);
}
// the same with the strip statistics of the output (NT, 64-wide k-tiles, three stages)
template <int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64) void gemm_bf16_dma_stats_kernel(const GemmArgs g) {
    gemm_bf16_dma_body<BM, BN, WM, WN, false, false, true, 3, 64, false, 0, 1>(g, blockIdx.x, blockIdx.z);
}
// input gradient of a 1x1 convolution (NN, 64-wide k-tiles, three stages) with the backward sums of the batch
// normalisation in front of it
template <int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64) void gemm_bf16_dma_bnbwd_kernel(const GemmArgs g, const BnBwdArgs bn) {
    gemm_bf16_dma_body<BM, BN, WM, WN, false, true, true, 3, 64, false, 0, 2>(g, blockIdx.x, 0, false, ConvArgs{}, bn);
}

// Persistent variant for problems of more than one round of 256x256 tiles (NT and NN, 32-wide k-tiles, three stages,
// eight waves): a block walks the output tiles b, b + gridDim, ... and treats their k-tiles as ONE stream, so the DMA
// ring never drains - while the last k-tiles of a tile are multiplied, the first ones of the block's next tile are
// already landing, and the epilogue's stores go out behind them.  What a tile boundary costs a block of the plain
// kernel (retiring, the next block's launch, its pipeline prologue) is gone: 95 -> 77 us on the plain product
// 8192 x 4096 x 1024.  The waits of the first k-tiles after a boundary count the epilogue's stores in (completion is in
// order): exact counts that spare them changed nothing, the stores are acknowledged quickly.  The epilogue patch
// cannot share the ring's LDS any more (the ring is live during the epilogue): it has 64 KB of its own behind the
// three stages, [32][64] floats per wave with the 16-byte chunks of a row swizzled by the row instead of padded.
// Results are bit-equal to the plain kernels' (same k order, same epilogue function).  Needs K % 64 == 0 (the two
// fragment sets alternate, a tile takes an even number of k-tiles), unbatched operands, a grid that is a multiple of 8
// (the tile order's XCD mapping).  Instantiated for 256x256 tiles only: 256x128 tiles on this loop load their 32-wide
// k-tiles as half lines and lose more than the boundaries give (90 against 71 us on 8192 x 3072 x 1024).
template <int BM, int BN, int WM, int WN, bool BKM, bool DROP>
__global__ __launch_bounds__(WM* WN * 64) void gemm_bf16_dma_persist_kernel(const GemmArgs g) {
    constexpr int NW = WM * WN, BK = 32, STAGES = 3;
    constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32;
    static_assert(TN == 2 && TM * TN > 2, "the epilogue patch holds two accumulator tiles side by side");
    using OpA = DmaOperand<BM, false, NW, BK>;
    using OpB = DmaOperand<BN, BKM, NW, BK>;
    constexpr int STAGE_BYTES = OpA::BYTES + OpB::BYTES;
    constexpr int LOADS = OpA::ROUNDS + OpB::ROUNDS;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int total = g.tiles_m * g.tiles_n, G = gridDim.x;
    const bf16* A = (const bf16*)g.A;
    const bf16* B = (const bf16*)g.B;
    const int KT = g.K / BK;

    OpA opa;
    OpB opb;
    FragReader<BM, TM, false, BK> fa;
    FragReader<BN, TN, BKM, BK> fb;
    fa.init(wm * WTM, lane);
    fb.init(wn * WTN, lane);
    struct Frags {
        bf16x8 a[2][TM], b[2][TN];
    };
    Frags f0, f1;
    f32x16 acc[TM][TN];

    // the stream: ki = index of the next k-tile to issue inside output tile issue_tile
    int issue_stage = 0, read_stage = 0, ki = 0, issue_tile = blockIdx.x;
    auto point_at = [&](int t) {
        int tm, tn;
        tile_coords(t, g.tiles_m, g.tiles_n, tm, tn);
        opa.init(A, g.lda, tm * BM, g.M, tid);
        opb.init(B, g.ldb, tn * BN, g.N, tid);
    };
    point_at(issue_tile);
    // before a k-tile is issued: move on to the block's next output tile, or (no tile left) stay on the last k-tile,
    // which is then fetched again and again into stages nobody reads
    auto prep_issue = [&]() {
        if (ki == KT) {
            if (issue_tile + G < total) {
                issue_tile += G;
                ki = 0;
                point_at(issue_tile);
            } else {
                ki = KT - 1;
            }
        }
        if (ki == KT - 1 && issue_tile + G >= total) {
            opa.stop();
            opb.stop();
        }
    };
    // MFMA m of step ks, then its share of ND DMA instructions into `dst` and of the fragment reads of `src` into
    // nf, each group fenced (see gemm_bf16_dma_body)
    auto placed_step = [&](const Frags& f, auto ks_c, auto nd_c, unsigned char* dst, auto reads_c, Frags& nf,
                           const unsigned char* src) {
        constexpr int ks = decltype(ks_c)::value, ND = decltype(nd_c)::value;
        constexpr bool READS = decltype(reads_c)::value;
        constexpr int NM = TM * TN, NF = 2 * (TM + TN), FM = NM - 2;
        static_for(
            [&](auto idx) {
                constexpr int m = decltype(idx)::value, i = m / TN, j = m % TN;
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.a[ks][i], f.b[ks][j], acc[i][j], 0, 0, 0);
                static_for(
                    [&](auto d) {
                        constexpr int k = (ND * m) / NM + decltype(d)::value;
                        if constexpr (k < OpA::ROUNDS) opa.template issue_one<k>(dst, wave);
                        else opb.template issue_one<k - OpA::ROUNDS>(dst + OpA::BYTES, wave);
                    },
                    std::make_integer_sequence<int, (ND * (m + 1)) / NM - (ND * m) / NM>{});
                if constexpr (READS && m < FM) {
                    static_for(
                        [&](auto r) {
                            constexpr int q = (NF * m) / FM + decltype(r)::value, fk = q / (TM + TN), t = q % (TM + TN);
                            if constexpr (t < TM) nf.a[fk][t] = fa.load(src, t, fk);
                            else nf.b[fk][t - TM] = fb.load(src + OpA::BYTES, t - TM, fk);
                        },
                        std::make_integer_sequence<int, (NF * (m + 1)) / FM - (NF * m) / FM>{});
                }
                __builtin_amdgcn_sched_barrier(0);
            },
            std::make_integer_sequence<int, NM>{});
    };
    // one k-tile: first half with the DMA instructions of the stream's k-tile two ahead, the wait for the k-tile
    // one ahead (in-order completion: whatever the epilogue stored before is acknowledged by then too), second half
    // with that k-tile's fragment reads
    auto body = [&](Frags& cur, Frags& nxt, auto reads_c) {
        prep_issue();
        unsigned char* dst = smem + issue_stage * STAGE_BYTES;
        issue_stage = issue_stage + 1 == STAGES ? 0 : issue_stage + 1;
        placed_step(cur, std::integral_constant<int, 0>{}, std::integral_constant<int, LOADS>{}, dst, std::false_type{}, nxt, smem);
        ++ki;
        asm volatile("" ::: "memory");
        wait_vmcnt_lgkm0<(STAGES - 2) * LOADS>();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const unsigned char* st = smem + read_stage * STAGE_BYTES;
        read_stage = read_stage + 1 == STAGES ? 0 : read_stage + 1;
        placed_step(cur, std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{}, dst, reads_c, nxt, st);
    };
    auto load_frags = [&](Frags& f, const unsigned char* st) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int i = 0; i < TM; ++i) f.a[ks][i] = fa.load(st, i, ks);
#pragma unroll
            for (int j = 0; j < TN; ++j) f.b[ks][j] = fb.load(st + OpA::BYTES, j, ks);
        }
    };

    // prologue of the stream
#pragma unroll
    for (int t = 0; t < STAGES - 1; ++t) {
        prep_issue();
        unsigned char* st = smem + issue_stage * STAGE_BYTES;
        opa.issue(st, wave);
        opb.issue(st + OpA::BYTES, wave);
        issue_stage = issue_stage + 1 == STAGES ? 0 : issue_stage + 1;
        ++ki;
    }
    asm volatile("" ::: "memory");
    wait_vmcnt_lgkm0<(STAGES - 2) * LOADS>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    float* patch = (float*)(smem + STAGES * STAGE_BYTES) + wave * (32 * 64);
    const int prow = lane >> 3, pchunk = lane & 7;
    // the two 16-byte chunks of a lane's eight columns, read in an order that keeps the eight lanes of a row on
    // eight different bank groups: lanes 0..3 of the row take their even chunk first, lanes 4..7 their odd one
    const int first_chunk = 2 * pchunk + (pchunk >> 2), second_chunk = 2 * pchunk + 1 - (pchunk >> 2);
    for (int tile = blockIdx.x; tile < total; tile += G) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
        // the tile's first fragments (the k-tile landed and was made visible by the last barrier before this point);
        // a tile's last k-tile does not fetch the next tile's, so that no fragment registers live through the epilogue
        load_frags(f0, smem + read_stage * STAGE_BYTES);
        read_stage = read_stage + 1 == STAGES ? 0 : read_stage + 1;
        for (int kt = 0; kt + 2 < KT; kt += 2) {
            body(f0, f1, std::true_type{});
            body(f1, f0, std::true_type{});
        }
        body(f0, f1, std::true_type{});
        body(f1, f0, std::false_type{});
        read_stage = read_stage == 0 ? STAGES - 1 : read_stage - 1;   // that k-tile is still to be read
        int tm, tn;
        tile_coords(tile, g.tiles_m, g.tiles_n, tm, tn);
        const int m0 = tm * BM + wm * WTM, n = tn * BN + wn * WTN + pchunk * 8;
        // the bias of the lane's eight columns once per tile; row offsets by addition (see gemm_bf16_dma_body)
        float b8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (g.bias && n < g.N) load_vec((const bf16*)g.bias + n, b8);
        int64_t ci = (int64_t)(m0 + prow) * g.ldc + n, xi = (int64_t)(m0 + prow) * g.ldaux + n;
        // the operand of the epilogue kinds that read one, fetched a patch ahead of its use (inside the epilogue only:
        // the main loop has no register to spare for it)
        const bf16* opnd = epilogue_operand(g);
        u32x4 opc[4], opn[4];
        auto fetch = [&](int i, u32x4 (&dst)[4]) {
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const int m = m0 + i * 32 + it * 8 + prow;
                dst[it] = u32x4{0u, 0u, 0u, 0u};
                if (opnd && m < g.M && n < g.N) dst[it] = *(const u32x4*)(opnd + (int64_t)m * g.ldaux + n);
            }
        };
        fetch(0, opc);
        // (static_for: a loop the compiler declines to unroll would index the accumulators dynamically, i.e. from scratch)
        static_for(
            [&](auto idx) {
                constexpr int i = decltype(idx)::value;
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int row = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3), col = h * 32 + (lane & 31);
                        patch[row * 64 + ((((col >> 2) ^ (row & 15)) << 2) | (col & 3))] = acc[i][h][r] * g.alpha;
                    }
                asm volatile("" ::: "memory");
                if constexpr (i + 1 < TM) fetch(i + 1, opn);
                static_for(
                    [&](auto it_c) {
                    constexpr int it = decltype(it_c)::value;
                    const int row = it * 8 + prow, m = m0 + i * 32 + row;
                    const f32x4 c1 = *(const f32x4*)(patch + row * 64 + ((first_chunk ^ (row & 15)) << 2));
                    const f32x4 c2 = *(const f32x4*)(patch + row * 64 + ((second_chunk ^ (row & 15)) << 2));
                    const f32x4 lo = pchunk < 4 ? c1 : c2, hi = pchunk < 4 ? c2 : c1;
                    float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    if (m < g.M && n < g.N) epilogue_vec8_at<DROP, true>(g, ci, xi, m, n, v, b8, opc[it]);
                    ci += 8 * (int64_t)g.ldc;
                    xi += 8 * (int64_t)g.ldaux;
                    },
                    std::make_integer_sequence<int, 4>{});
                asm volatile("" ::: "memory");
#pragma unroll
                for (int it = 0; it < 4; ++it) opc[it] = opn[it];
            },
            std::make_integer_sequence<int, TM>{});
    }
    wait_vmcnt_lgkm0<0>();   // the k-tiles issued past the end of the stream land before the block leaves
}

// 3x3 convolution as an implicit GEMM: forward (BKM = false: y = patches(x) W^T) and input gradient
// (BKM = true: dx = patches(dy) W_flipped) on the same main loop, operands gathered by the loaders.
template <int BM, int BN, int WM, int WN, bool BKM, int STAGES, bool STATS = false>
__global__ __launch_bounds__(WM* WN * 64) void conv3x3_bf16_igemm_kernel(const GemmArgs g, const ConvArgs cv) {
    gemm_bf16_dma_body<BM, BN, WM, WN, false, BKM, true, STAGES, 64, false, BKM ? 2 : 1, STATS ? 1 : 0>(g, blockIdx.x, 0, false, cv);
}
// the input gradient with the backward sums of the batch normalisation in front of the convolution
template <int BM, int BN, int WM, int WN, int STAGES>
__global__ __launch_bounds__(WM* WN * 64) void conv3x3_bf16_igemm_bnbwd_kernel(const GemmArgs g, const ConvArgs cv, const BnBwdArgs bn) {
    gemm_bf16_dma_body<BM, BN, WM, WN, false, true, true, STAGES, 64, false, 2, 2>(g, blockIdx.x, 0, false, cv, bn);
}

// Several independent problems of one kind in a single launch (the four weight-gradient GEMMs
// of a transformer layer: each alone has too few output tiles to fill 256 CUs).
constexpr int GROUP_MAX = 16;
struct GroupedArgs {
    GemmArgs p[GROUP_MAX];
    int first_block[GROUP_MAX + 1];
    int count;
};
// CONVB: some problems of the group read their B operand as the patch matrix of a 3x3 convolution
template <int BM, int BN, int WM, int WN, bool AKM, bool BKM, bool DB, int STAGES, bool CONVB = false>
__global__ __launch_bounds__(WM* WN * 64) void gemm_bf16_dma_grouped_kernel(const GroupedArgs G) {
    // The tiles of all problems form one list; an XCD takes a contiguous stretch of it, so its
    // resident blocks are a few wide rectangles of one or two problems (few distinct operand
    // panels in its L2) rather than a narrow slice of every problem.
    const int lid = xcd_contiguous(blockIdx.x, G.first_block[G.count]);
    int pi = 0;
    while (pi + 1 < G.count && lid >= G.first_block[pi + 1]) ++pi;
    // compiler-visible DMA here: the lock step it forces on the waves keeps the three resident blocks of a CU
    // on the same operand panels (459 instead of 720 MiB read per launch at the same kernel speed; the stage
    // gains half a percent with the second stream running)
    if constexpr (CONVB) {
        if (G.p[pi].conv_c > 0) {
            gemm_bf16_dma_body<BM, BN, WM, WN, AKM, BKM, DB, STAGES, 32, true, 3>(G.p[pi], lid - G.first_block[pi], 0, true);
            return;
        }
    }
    gemm_bf16_dma_body<BM, BN, WM, WN, AKM, BKM, DB, STAGES, 32, true>(G.p[pi], lid - G.first_block[pi], 0, true);
}

// =========================================================================================
// fp32 kernel: 128x128x16 tiles, 4 waves (2x2), LDS k-major with padded rows.
// =========================================================================================
// TILE = BM = BN: 128 (wave tile 64x64), or 64 (wave tile 32x32) for problems with so few 128x128 tiles that most CUs
// would hold one block, i.e. one wave per SIMD with nobody to cover its waits for the next k-tile.  Every element adds
// up its contraction in the same order on both.
// BN = 32 (TILE 64): 64x32 tiles of two waves, and KG > 1: KG groups of waves share a tile; group j takes the k-tiles
// j, j + KG, ... through LDS buffers of its own and the groups' partial tiles are added in group order at the end --
// for problems that have fewer than two 64x64 tiles per CU and a long contraction (a different, equally fixed order of
// additions: the shape alone decides).
// (block_id: the block's index among the problem's tiles; logical_id: it is not a hardware block id, so the tile order
// takes it as it is instead of undoing the round-robin over the XCDs)

// one k-tile of an operand, ROWS x BK: global -> registers (zeros past the operand's rows and past the contraction, so
// a group whose share is one k-tile shorter adds nothing), registers -> LDS [k][row]
template <int ROWS, int BK, int NT, int CH>
__device__ __forceinline__ void f32_gload(const float* base, int64_t ld, int row0, int rows, int k0, int K, bool tr, int tid,
                                          f32x4 (&r)[CH]) {
    constexpr int RQ = ROWS / 4;   // chunks along a row-contiguous (transposed) tile row
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        const int c = tid + i * NT;
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        if (!tr) {
            const int row = c >> 2, kq = c & 3;
            if (row0 + row < rows && k0 + kq * 4 < K) v = *(const f32x4*)(base + (int64_t)(row0 + row) * ld + k0 + kq * 4);
        } else {
            const int k = c / RQ, rq = c % RQ;
            if (row0 + rq * 4 < rows && k0 + k < K) v = *(const f32x4*)(base + (int64_t)(k0 + k) * ld + row0 + rq * 4);
        }
        r[i] = v;
    }
}
template <int ROWS, int LD, int NT, int CH>
__device__ __forceinline__ void f32_sstore(float* lds, bool tr, int tid, const f32x4 (&r)[CH]) {
    constexpr int RQ = ROWS / 4;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        const int c = tid + i * NT;
        if (!tr) {
            const int row = c >> 2, kq = c & 3;
#pragma unroll
            for (int e = 0; e < 4; ++e) lds[(kq * 4 + e) * LD + row] = r[i][e];
        } else {
            const int k = c / RQ, rq = c % RQ;
            *(f32x4*)(lds + k * LD + rq * 4) = r[i];
        }
    }
}

template <bool TA, bool TB, int TILE, int KG = 1, int BN = TILE>
__device__ __forceinline__ void gemm_f32_body(const GemmArgs& g, const int block_id, const int batch_id, const bool logical_id) {
    static_assert(BN == TILE || (TILE == 64 && BN == 32), "tiles: 128x128, 64x64, 64x32");
    static_assert(KG == 1 || TILE == 64, "the contraction is split over wave groups on the small tiles only");
    constexpr int BM = TILE, BK = 16, LDA = BM + 4, LDB = BN + 4;
    constexpr int WTM = TILE / 2, WTN = BN == TILE ? TILE / 2 : BN;   // wave tile
    constexpr int WN = BN / WTN, NT = 64 * (BM / WTM) * WN;           // waves along N, threads of a group
    constexpr int TFM = WTM / 32, TFN = WTN / 32;                     // 32x32 accumulator tiles of a wave
    constexpr int CHA = BM * BK / 4 / NT, CHB = BN * BK / 4 / NT;     // 16-byte chunks of an operand tile per thread
    constexpr int GROUP_LDS = 2 * BK * (LDA + LDB);                   // two stages of A, then two of B
    __shared__ __attribute__((aligned(16))) float lds_all[KG][GROUP_LDS];
    const int grp = KG == 1 ? 0 : threadIdx.x / NT;
    const int tid = threadIdx.x % NT, lane = tid & 63, wave = tid >> 6;
    float* const As = lds_all[grp];
    float* const Bs = lds_all[grp] + 2 * BK * LDA;
    const int wm = WN == 2 ? wave >> 1 : wave, wn = WN == 2 ? wave & 1 : 0;
    int tile_m, tile_n;
    if (logical_id) panel_coords(block_id, g.tiles_m, g.tiles_n, tile_m, tile_n);
    else tile_coords(block_id, g.tiles_m, g.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int b1 = batch_id / g.nb2, b2 = batch_id % g.nb2;
    const float* A = (const float*)g.A + b1 * g.sA1 + b2 * g.sA2;
    const float* B = (const float*)g.B + b1 * g.sB1 + b2 * g.sB2;
    const int64_t coff = b1 * g.sC1 + b2 * g.sC2;

    f32x4 ra[CHA], rb[CHB];
    f32x16 acc[TFM][TFN];
#pragma unroll
    for (int i = 0; i < TFM; ++i)
#pragma unroll
        for (int j = 0; j < TFN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // every group runs the same number of rounds (the barriers are the block's); round kt of group grp is k-tile
    // kt * KG + grp
    const int KT = ((g.K + BK - 1) / BK + KG - 1) / KG;
    f32_gload<BM, BK, NT, CHA>(A, g.lda, m0, g.M, grp * BK, g.K, TA, tid, ra);
    f32_gload<BN, BK, NT, CHB>(B, g.ldb, n0, g.N, grp * BK, g.K, TB, tid, rb);
    f32_sstore<BM, LDA, NT, CHA>(As, TA, tid, ra);
    f32_sstore<BN, LDB, NT, CHB>(Bs, TB, tid, rb);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        const bool more = kt + 1 < KT;
        if (more) {
            f32_gload<BM, BK, NT, CHA>(A, g.lda, m0, g.M, ((kt + 1) * KG + grp) * BK, g.K, TA, tid, ra);
            f32_gload<BN, BK, NT, CHB>(B, g.ldb, n0, g.N, ((kt + 1) * KG + grp) * BK, g.K, TB, tid, rb);
        }
        const float* as = As + cur * BK * LDA;
        const float* bs = Bs + cur * BK * LDB;
#pragma unroll
        for (int ks = 0; ks < BK / 2; ++ks) {
            float af[TFM], bfr[TFN];
            const int kk = ks * 2 + (lane >> 5);
#pragma unroll
            for (int i = 0; i < TFM; ++i) af[i] = as[kk * LDA + wm * WTM + i * 32 + (lane & 31)];
#pragma unroll
            for (int j = 0; j < TFN; ++j) bfr[j] = bs[kk * LDB + wn * WTN + j * 32 + (lane & 31)];
#pragma unroll
            for (int i = 0; i < TFM; ++i)
#pragma unroll
                for (int j = 0; j < TFN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bfr[j], acc[i][j], 0, 0, 0);
        }
        if (more) {
            f32_sstore<BM, LDA, NT, CHA>(As + (cur ^ 1) * BK * LDA, TA, tid, ra);
            f32_sstore<BN, LDB, NT, CHB>(Bs + (cur ^ 1) * BK * LDB, TB, tid, rb);
        }
        __syncthreads();
    }
    if constexpr (KG > 1) {
        // partial tiles of groups 1 .. KG-1 go through the groups' own (now idle) operand buffers; group 0 adds them up
        // in group order
        static_assert(TFM == 1 && TFN == 1 && GROUP_LDS >= 16 * NT, "a group's operand buffers hold its partial tile");
        if (grp > 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r) lds_all[grp][r * NT + tid] = acc[0][0][r];
        }
        __syncthreads();
        if (grp > 0) return;
#pragma unroll
        for (int j = 1; j < KG; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[0][0][r] += lds_all[j][r * NT + tid];
    }
#pragma unroll
    for (int i = 0; i < TFM; ++i)
#pragma unroll
        for (int j = 0; j < TFN; ++j) {
            const int n = n0 + wn * WTN + j * 32 + (lane & 31);
            if (n >= g.N) continue;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * WTM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (m < g.M) epilogue_elem<float>(g, coff, coff, m, n, acc[i][j][r]);
            }
        }
}

template <bool TA, bool TB, int TILE = 128>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const GemmArgs g) {
    gemm_f32_body<TA, TB, TILE>(g, blockIdx.x, blockIdx.z, false);
}
// small tiles (64 x BN), the contraction dealt to KG groups of waves
template <bool TA, bool TB, int KG, int BN>
__global__ __launch_bounds__(4 * BN * KG) void gemm_f32_ksplit_kernel(const GemmArgs g) {
    gemm_f32_body<TA, TB, 64, KG, BN>(g, blockIdx.x, blockIdx.z, false);
}
// several unbatched problems in one launch (the weight gradients of an fp32 layer: the smallest has 144 tiles of 64x64)
template <bool TA, bool TB, int TILE>
__global__ __launch_bounds__(256) void gemm_f32_grouped_kernel(const GroupedArgs G) {
    const int lid = xcd_contiguous(blockIdx.x, G.first_block[G.count]);
    int pi = 0;
    while (pi + 1 < G.count && lid >= G.first_block[pi + 1]) ++pi;
    gemm_f32_body<TA, TB, TILE>(G.p[pi], lid - G.first_block[pi], 0, true);
}

