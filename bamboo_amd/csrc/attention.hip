// Fused masked softmax-attention for gfx950, bf16, head dimension 64, 32 or 128: forward and the two
// backward kernels (dK/dV and dQ).  No [batch, heads, seq, seq] tensor ever reaches HBM; the
// forward keeps one fp32 log-sum-exp per (batch, head, query) for the backward.
//
// Stands in for MultiHeadedAttention.attention of the reference
// (DeepSpeedExamples/pipeline_parallelism/transformer.py:117-127: softmax(QK^T/sqrt(d) with
// masked_fill(mask == 0, -1e9)) V) and for its autograd backward.
//
// Layout.  Q, K, V of head j are the 64-wide column slices at j*64 of the three thirds of the
// [rows, 3*hidden] projection buffer; the context goes to columns j*64 of a [rows, hidden]
// buffer.  Each wave owns 32 rows (queries in forward / dQ, keys in dK/dV) and keeps one score
// COLUMN per lane: scores are produced transposed (S^T = K Q^T), so the softmax reductions over
// keys are in-lane plus one cross-half shuffle, and P^T comes out of the accumulators already
// in the register layout the next MFMA wants as its B operand.  With 32-wide heads (HP = 2) a block
// owns a PAIR of neighbouring heads, whose columns together are one 64-wide slice: the tiles in LDS,
// their loads and the fragment layout are those of one 64-wide head, every product takes the k-steps
// (scores) or the output tile (context, gradients) of its head, the softmax runs once per head.
// Operands that are contracted
// over their row index (V in O = PV, Q and dO in dK/dV, K in dQ) are read from LDS with
// ds_read_b64_tr_b16.  Tiles travel global -> LDS by DMA (global_load_lds_dwordx4),
// double-buffered.  All reductions have a fixed order: results are reproducible bit for bit.
#include "common.h"

typedef __attribute__((address_space(3))) void lds_ptr_t;
typedef const __attribute__((address_space(1))) void gbl_ptr_t;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;

struct AttnArgs {
    const bf16* q; const bf16* k; const bf16* v;   // head 0 of batch 0; row stride ld_qkv
    const bf16* o; const bf16* d_o;                // [rows, hidden] context and its gradient
    bf16* out;                                     // forward: context
    bf16* dq; bf16* dk; bf16* dv;                  // backward outputs, row stride ld_dqkv
    float* lse;                                    // [batch, heads, seq], log2 domain
    float* delta;                                  // [batch, heads, seq], rowsum(dO * O)
    const int32_t* key_len;
    int64_t ld_qkv, ld_o, ld_dqkv;
    int batch, heads, seq, mask;
    float scale_log2;                              // log2(e) / sqrt(d)
    float scale;                                   // 1 / sqrt(d)
    DropKey drop;                                  // dropout on the probabilities (thresh 0: none)
};
// index of probability (b, head, q, kv) in the [batch, heads, seq, seq] tensor that is never stored
__device__ __forceinline__ uint64_t prob_index(const AttnArgs& a, int b, int head, int q) {
    return ((uint64_t)(b * a.heads + head) * a.seq + q) * a.seq;
}

// Global -> LDS transfers (16 or 4 bytes per lane; the LDS target is M0 + lane * size), issued as
// inline assembly: while the compiler sees such a load in flight it turns every wait for an LDS
// read into lgkmcnt(0).  Unseen, fragment waits keep their exact counts; the kernels wait for
// these loads explicitly (wait_vm) before each barrier, as they always did.
__device__ __forceinline__ void dma16(const void* src, const unsigned char* lds_dst) {
    const unsigned m0 = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)(lds_ptr_t*)lds_dst);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(m0), "v"(src) : "m0");
}
__device__ __forceinline__ void dma4(const void* src, const unsigned char* lds_dst) {
    const unsigned m0 = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)(lds_ptr_t*)lds_dst);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(m0), "v"(src) : "m0");
}

// ---- LDS tile format: [rows][64] bf16, 128 B per row, 16-byte chunk c of row r at slot c ^ fsw(r)
__device__ __forceinline__ int fsw(int r) { return (((r >> 1) & 1) << 2) | (((r >> 2) & 1) << 1) | ((r >> 3) & 1); }

// one wave-instruction moves 8 rows; instruction `idx` of a tile covers rows idx*8 .. idx*8+7
__device__ __forceinline__ void dma_rows8(const bf16* gbase, int64_t ld, int row0, int last_row, unsigned char* tile,
                                          int idx, int lane) {
    const int r = idx * 8 + (lane >> 3);
    const int c = (lane & 7) ^ fsw(r);
    const int gr = min(row0 + r, last_row);
    dma16(gbase + (int64_t)gr * ld + c * 8, tile + idx * 1024);
}
// Whole 64-row tile: this wave's two instructions (row groups wave and wave + 4).  Full tiles
// take a wave-uniform base plus the lane's fixed offset; only a tile that reaches past the last
// row pays for per-lane clamping.
struct LaneOff { uint32_t o0, o1; };
__device__ __forceinline__ LaneOff lane_off(int64_t ld, int wave, int lane) {
    const int r0 = wave * 8 + (lane >> 3), r1 = r0 + 32;
    return {(uint32_t)(r0 * ld + (((lane & 7) ^ fsw(r0)) << 3)), (uint32_t)(r1 * ld + (((lane & 7) ^ fsw(r1)) << 3))};
}
__device__ __forceinline__ void dma_tile64(const bf16* gbase, int64_t ld, int row0, int last_row, unsigned char* tile,
                                           int wave, int lane, LaneOff lo) {
    if (row0 + 63 <= last_row) {
        const bf16* g = gbase + (int64_t)row0 * ld;
        dma16(g + lo.o0, tile + wave * 1024);
        dma16(g + lo.o1, tile + (wave + 4) * 1024);
    } else {
        dma_rows8(gbase, ld, row0, last_row, tile, wave, lane);
        dma_rows8(gbase, ld, row0, last_row, tile, wave + 4, lane);
    }
}
// 4-byte variant for the per-row fp32 statistics: 64 consecutive floats
__device__ __forceinline__ void dma_f32x64(const float* gbase, int idx0, int last, unsigned char* dst, int lane) {
    const int i = min(idx0 + lane, last);
    dma4(gbase + i, dst);
}

// A/B fragment along the contiguous (feature) dimension: lane (r = lane%32, kg = lane/32) gets
// features ks*16 + kg*8 .. +8 of tile row row0 + r
__device__ __forceinline__ bf16x8 frag_kc(const unsigned char* tile, int row0, int ks, int lane) {
    const int r = row0 + (lane & 31);
    const int chunk = ks * 2 + (lane >> 5);
    return *(const bf16x8*)(tile + r * 128 + ((chunk ^ fsw(r)) << 4));
}
// A fragment contracted over tile ROWS: lane (c = lane%32, kg = lane/32) gets, for feature column
// col0 + c, the rows rbase + 4kg + {0..3} and rbase + 8 + 4kg + {0..3}: the row order in which a
// 32x32 accumulator column sits in registers 0..7 of a lane
__device__ __forceinline__ bf16x8 frag_tr(const unsigned char* tile, int rbase, int col0, int lane) {
    const int j = lane & 15;
    const int col = col0 + ((lane >> 4) & 1) * 16 + 4 * (j & 3);
    const int r0 = rbase + 4 * (lane >> 5) + (j >> 2);
    const int r1 = r0 + 8;
    const unsigned char* p0 = tile + r0 * 128 + (((col >> 3) ^ fsw(r0)) << 4) + (col & 7) * 2;
    const unsigned char* p1 = tile + r1 * 128 + (((col >> 3) ^ fsw(r1)) << 4) + (col & 7) * 2;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p0);
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p1);
    s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8, v);
}
// registers 8*half .. 8*half+7 of a 32x32 accumulator as a bf16 B fragment
__device__ __forceinline__ bf16x8 pack_acc(const f32x16& a, int half) {
    bf16x8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (__bf16)a[half * 8 + e];
    return v;
}
// row index (0..31) that register r of a 32x32 accumulator holds in this lane
__device__ __forceinline__ int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }
// Dropout over the sixteen accumulator registers of a lane whose rows acc_row(r, lane) are consecutive probability
// indices from `base` on: registers 4g .. 4g + 3 hold four neighbouring indices, i.e. two hash pairs when the first is
// even (every case with an even sequence length).  Kept values are scaled, dropped ones zeroed.
__device__ __forceinline__ void drop_acc_rows(const DropKey& k, uint64_t base, int lane, f32x16& v) {
    const bool even = (base & 1) == 0;   // 8 g + 4 (lane >> 5) is even
    if (k.small && even) {               // the rule: fewer than 2^32 probabilities, even sequence length
        const uint32_t p0 = ((uint32_t)base >> 1) + 2 * (lane >> 5);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const uint32_t x0 = bb_dropout_pair_bits32(k.k0, k.k1, p0 + 4 * g), x1 = bb_dropout_pair_bits32(k.k0, k.k1, p0 + 4 * g + 1);
            v[4 * g] = bb_keep_even(x0, k.thresh) ? v[4 * g] * k.scale : 0.f;
            v[4 * g + 1] = bb_keep_odd(x0, k.thresh) ? v[4 * g + 1] * k.scale : 0.f;
            v[4 * g + 2] = bb_keep_even(x1, k.thresh) ? v[4 * g + 2] * k.scale : 0.f;
            v[4 * g + 3] = bb_keep_odd(x1, k.thresh) ? v[4 * g + 3] * k.scale : 0.f;
        }
        return;
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const uint64_t i0 = base + 8 * g + 4 * (lane >> 5);
#pragma unroll
        for (int e = 0; e < 4; ++e)
            v[4 * g + e] = bb_dropout_keep(k.k0, k.k1, k.thresh, i0 + e) ? v[4 * g + e] * k.scale : 0.f;
    }
}

template <int N> __device__ __forceinline__ void wait_vm() {
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (0 << 8) | ((N >> 4) << 14));
}
__device__ __forceinline__ void block_sync() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// number of leading keys a query may see (mask applied as in the reference: keep kv < limit)
__device__ __forceinline__ int kv_limit(const AttnArgs& a, int b, int q) {
    if (a.mask == BB_MASK_CAUSAL) return min(a.seq, q + 1);
    if (a.mask == BB_MASK_KEY_PADDING) return min(a.seq, a.key_len[b]);
    return a.seq;
}

// Block -> (row block, batch*head) map for a 1-D grid of 8 * ceil(nbh / 8) * nblk blocks.  The
// hardware deals consecutive block ids round-robin over the 8 XCDs, so the low three bits of
// the id pick the XCD.  Each XCD is given whole (batch, head) pairs - all their row blocks, so
// the pair's K and V stay in that XCD's L2 - and, under a causal mask, the same mix of long and
// short blocks as every other XCD, longest first (rank 0 = most work).
struct BlockMap { int rank, bh; };
__device__ __forceinline__ BlockMap map_block(int nbh) {
    const int per_xcd = (nbh + 7) >> 3;
    const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
    return {j / per_xcd, (j % per_xcd) * 8 + xcd};
}
static unsigned attn_grid(int seq, int nbh) { return (unsigned)(8 * ((nbh + 7) / 8) * ((seq + 127) / 128)); }

// =========================================================================================
// forward: block = 128 queries (4 waves x 32), loop over 64-key tiles
// =========================================================================================
// HP: heads per block (1: one head, 2: a pair of 32-wide heads); NPAN: 64-wide column panels of a head (1; 2 for
// 128-wide heads, HP = 1: a tile in LDS is then two [64][64] panels behind each other, each in the format above);
// KS k-steps of a head's scores, DT 32-wide output tiles of a head
template <bool DROP, int HP, int NPAN = 1>
__global__ __launch_bounds__(256, (!DROP && NPAN == 1 && HP == 1) ? 4 : 2) void attn_fwd_kernel(const AttnArgs a) {
    static_assert(HP == 1 || NPAN == 1, "pairs of heads are 32 wide");
    constexpr int KS = 4 * NPAN / HP, DT = 2 * NPAN / HP, TILE = NPAN * 8192;
    __shared__ __attribute__((aligned(16))) unsigned char smem[2 * 2 * TILE];  // 2 stages x (K, V)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int groups = a.heads / HP;
    const BlockMap bm = map_block(a.batch * groups);
    if (bm.bh >= a.batch * groups) return;
    const int qb = (a.seq + 127) / 128 - 1 - bm.rank;  // long (late) query blocks first
    const int b = bm.bh / groups, hg = bm.bh % groups, head0 = hg * HP;
    const int64_t row_base = (int64_t)b * a.seq;
    const bf16* Q = a.q + row_base * a.ld_qkv + hg * (64 * NPAN);
    const bf16* K = a.k + row_base * a.ld_qkv + hg * (64 * NPAN);
    const bf16* V = a.v + row_base * a.ld_qkv + hg * (64 * NPAN);
    const int q0 = qb * 128 + wave * 32;
    const int myq = q0 + (lane & 31);
    const int last = a.seq - 1;

    // block-wide key range
    int kv_end = a.seq;
    if (a.mask == BB_MASK_CAUSAL) kv_end = min(a.seq, qb * 128 + 128);
    else if (a.mask == BB_MASK_KEY_PADDING) kv_end = min(a.seq, a.key_len[b]);
    const int ntiles = (kv_end + 63) / 64;
    const int my_limit = kv_limit(a, b, myq);
    const int wave_min_limit = kv_limit(a, b, q0);  // limits grow with the query index

    bf16x8 qf[4 * NPAN];
    {
        const bf16* qp = Q + (int64_t)min(myq, last) * a.ld_qkv + (lane >> 5) * 8;
#pragma unroll
        for (int ks = 0; ks < 4 * NPAN; ++ks) qf[ks] = *(const bf16x8*)(qp + ks * 16);
    }
    f32x16 o[2 * NPAN];
#pragma unroll
    for (int t = 0; t < 2 * NPAN; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[t][r] = 0.f;
    float m[HP], lsum[HP];
#pragma unroll
    for (int hh = 0; hh < HP; ++hh) {
        m[hh] = -INFINITY;
        lsum[hh] = 0.f;
    }

    const LaneOff lo = lane_off(a.ld_qkv, wave, lane);
    auto issue = [&](int t) {
        unsigned char* st = smem + (t & 1) * (2 * TILE);
        const int kv0 = t * 64;
#pragma unroll
        for (int p = 0; p < NPAN; ++p) {
            dma_tile64(K + p * 64, a.ld_qkv, kv0, last, st + p * 8192, wave, lane, lo);
            dma_tile64(V + p * 64, a.ld_qkv, kv0, last, st + TILE + p * 8192, wave, lane, lo);
        }
    };

    if (ntiles > 0) issue(0);
    for (int t = 0; t < ntiles; ++t) {
        asm volatile("" ::: "memory");
        if (t + 1 < ntiles) {
            issue(t + 1);
            wait_vm<4 * NPAN>();
        } else {
            wait_vm<0>();
        }
        block_sync();
        const unsigned char* kt = smem + (t & 1) * (2 * TILE);
        const unsigned char* vt = kt + TILE;
        const int kv0 = t * 64;
        // waves whose queries all precede this tile have nothing to add (causal)
        const bool active = !(a.mask == BB_MASK_CAUSAL && kv0 > q0 + 31);
        if (active) {
#pragma unroll
          for (int hh = 0; hh < HP; ++hh) {
            f32x16 s[2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
#pragma unroll
                for (int r = 0; r < 16; ++r) s[u][r] = 0.f;
#pragma unroll
                for (int k = 0; k < KS; ++k) {
                    const int ks = hh * KS + k;   // k-step ks: panel ks / 4, step ks % 4 inside it
                    s[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_kc(kt + (ks >> 2) * 8192, u * 32, ks & 3, lane), qf[ks], s[u], 0, 0, 0);
                }
            }
            // running max on the raw scores (the scale is positive), masking only on tiles that
            // reach past the first key some query of this wave may not see
            const bool need_mask = kv0 + 64 > wave_min_limit;
            float tmax = -INFINITY;
            if (need_mask) {
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int kv = kv0 + u * 32 + acc_row(r, lane);
                        s[u][r] = kv < my_limit ? s[u][r] : -INFINITY;
                    }
            }
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, s[u][r]);
            tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64)) * a.scale_log2;
            const float mnew = fmaxf(m[hh], tmax);
            const float msafe = mnew == -INFINITY ? 0.f : mnew;
            const float alpha = __builtin_amdgcn_exp2f(m[hh] - msafe);  // m = -inf -> 0
            float psum = 0.f;
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float p = __builtin_amdgcn_exp2f(fmaf(s[u][r], a.scale_log2, -msafe));
                    s[u][r] = p;
                    psum += p;
                }
            lsum[hh] = lsum[hh] * alpha + psum;
            m[hh] = mnew;
            if (DROP && a.drop.thresh) {   // the normaliser takes every probability, the context only the kept ones
                const uint64_t base = prob_index(a, b, head0 + hh, min(myq, last)) + kv0;
#pragma unroll
                for (int u = 0; u < 2; ++u) drop_acc_rows(a.drop, base + u * 32, lane, s[u]);
            }
            if (__any(alpha != 1.0f)) {  // wave-uniform: once the maxima have settled nothing is rescaled
#pragma unroll
                for (int d = 0; d < DT; ++d)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o[hh * DT + d][r] *= alpha;
            }
            // O^T += V^T P^T
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                const bf16x8 pf = pack_acc(s[kk >> 1], kk & 1);
#pragma unroll
                for (int d = 0; d < DT; ++d) {
                    const int dt = hh * DT + d;   // output tile dt: panel dt / 2, columns (dt % 2) * 32 inside it
                    o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_tr(vt + (dt >> 1) * 8192, kk * 16, (dt & 1) * 32, lane), pf, o[dt], 0, 0, 0);
                }
            }
          }
        }
        block_sync();
    }
    float inv[HP];
#pragma unroll
    for (int hh = 0; hh < HP; ++hh) {
        lsum[hh] += __shfl_xor(lsum[hh], 32, 64);
        inv[hh] = lsum[hh] > 0.f ? 1.0f / lsum[hh] : 0.f;
    }
    if (myq < a.seq) {
        bf16* op = a.out + (row_base + myq) * a.ld_o + hg * (64 * NPAN);
#pragma unroll
        for (int dt = 0; dt < 2 * NPAN; ++dt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int d = dt * 32 + 8 * g4 + 4 * (lane >> 5);
                const float iv = inv[dt / DT];
                u32x2 w = {pack2bf(o[dt][g4 * 4] * iv, o[dt][g4 * 4 + 1] * iv),
                           pack2bf(o[dt][g4 * 4 + 2] * iv, o[dt][g4 * 4 + 3] * iv)};
                *(u32x2*)(op + d) = w;
            }
#pragma unroll
        for (int hh = 0; hh < HP; ++hh)
            if (lane < 32) a.lse[((int64_t)b * a.heads + head0 + hh) * a.seq + myq] = m[hh] + log2f(lsum[hh]);
    }
}

// =========================================================================================
// backward dK, dV: block = 128 keys (4 waves x 32), loop over 64-query tiles
// =========================================================================================
// NPAN = 2 (128-wide heads): a block accumulates dK and dV for ONE 64-wide half `fh` of the head's columns (the grid
// has two blocks per head and key block); scores and dP take the full 128 columns in both, i.e. are made twice -- a wave
// that held all four output tiles of dK and of dV next to K, V, S and dP would need more registers than it has.
template <bool DROP, int HP, int NPAN = 1>
__global__ __launch_bounds__(256, 2) void attn_bwd_dkv_kernel(const AttnArgs a) {
    static_assert(HP == 1 || NPAN == 1, "pairs of heads are 32 wide");
    constexpr int KS = 4 * NPAN / HP, DT = 2 / HP, TILE = NPAN * 8192;
    // 2 stages x (Q tile, dO tile: 8 KiB per panel, lse 256 B per head, delta 256 B per head); two panels: more than the
    // 64 KiB a kernel may declare, so the launch brings it
    constexpr int STAGE = 2 * TILE + 512 * HP;
    __shared__ __attribute__((aligned(16))) unsigned char smem_fixed[NPAN == 1 ? 2 * STAGE : 16];
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_launch[];
    unsigned char* smem = NPAN == 1 ? smem_fixed : smem_launch;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int groups = a.heads / HP;
    const BlockMap bm = map_block(a.batch * groups * NPAN);
    if (bm.bh >= a.batch * groups * NPAN) return;
    const int kb = bm.rank;  // early key blocks are seen by the most queries
    const int fh = bm.bh % NPAN, bg = bm.bh / NPAN;
    const int b = bg / groups, hg = bg % groups, head0 = hg * HP;
    const int64_t row_base = (int64_t)b * a.seq;
    const bf16* Q = a.q + row_base * a.ld_qkv + hg * (64 * NPAN);
    const bf16* K = a.k + row_base * a.ld_qkv + hg * (64 * NPAN);
    const bf16* V = a.v + row_base * a.ld_qkv + hg * (64 * NPAN);
    const bf16* DO = a.d_o + row_base * a.ld_o + hg * (64 * NPAN);
    // the statistics of the block's heads lie behind each other: [batch, heads, seq]
    const float* LSE = a.lse + ((int64_t)b * a.heads + head0) * a.seq;
    const float* DELTA = a.delta + ((int64_t)b * a.heads + head0) * a.seq;
    const int kv0 = kb * 128 + wave * 32;
    const int mykv = kv0 + (lane & 31);
    const int last = a.seq - 1;
    const int pad_limit = a.mask == BB_MASK_KEY_PADDING ? min(a.seq, a.key_len[b]) : a.seq;

    // query range that can see keys of this block
    const int q_begin = a.mask == BB_MASK_CAUSAL ? (kb * 128) / 64 : 0;  // first 64-query tile
    // a block whose 128 keys are all padding has nothing to accumulate: it only stores its zeros
    const int ntiles = kb * 128 >= pad_limit ? 0 : (a.seq + 63) / 64;

    bf16x8 kf[4 * NPAN], vf[4 * NPAN];
    {
        const int64_t off = (int64_t)min(mykv, last) * a.ld_qkv + (lane >> 5) * 8;
#pragma unroll
        for (int ks = 0; ks < 4 * NPAN; ++ks) {
            kf[ks] = *(const bf16x8*)(K + off + ks * 16);
            vf[ks] = *(const bf16x8*)(V + off + ks * 16);
        }
    }
    f32x16 dk[2], dv[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) dk[t][r] = dv[t][r] = 0.f;

    const LaneOff lo = lane_off(a.ld_qkv, wave, lane), lo_o = lane_off(a.ld_o, wave, lane);
    auto issue = [&](int t, int slot) {
        unsigned char* st = smem + slot * STAGE;
        const int qs = t * 64;
#pragma unroll
        for (int p = 0; p < NPAN; ++p) {
            dma_tile64(Q + p * 64, a.ld_qkv, qs, last, st + p * 8192, wave, lane, lo);
            dma_tile64(DO + p * 64, a.ld_o, qs, last, st + TILE + p * 8192, wave, lane, lo_o);
        }
        // one extra load for waves 0 and 1 (one head), for all four waves (a pair): lse of the heads, then delta
        if constexpr (HP == 1) {
            if (wave == 0) dma_f32x64(LSE, qs, last, st + 2 * TILE, lane);
            if (wave == 1) dma_f32x64(DELTA, qs, last, st + 2 * TILE + 256, lane);
        } else {
            const float* src = (wave >> 1 ? DELTA : LSE) + (int64_t)(wave & 1) * a.seq;
            dma_f32x64(src, qs, last, st + 2 * TILE + (wave >> 1) * 512 + (wave & 1) * 256, lane);
        }
    };

    if (q_begin < ntiles) issue(q_begin, 0);
    for (int t = q_begin; t < ntiles; ++t) {
        const int slot = (t - q_begin) & 1;
        asm volatile("" ::: "memory");
        if (t + 1 < ntiles) {
            issue(t + 1, slot ^ 1);
            // the waves with an extra load wait for one more newer load than the others
            if (HP == 2 || wave < 2) wait_vm<4 * NPAN + 1>(); else wait_vm<4 * NPAN>();
        } else {
            wait_vm<0>();
        }
        block_sync();
        const unsigned char* qt = smem + slot * STAGE;
        const unsigned char* dot = qt + TILE;
        const float* lse_all = (const float*)(qt + 2 * TILE);
        const float* del_all = lse_all + 64 * HP;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int qs = t * 64 + u * 32;
            if (a.mask == BB_MASK_CAUSAL && qs + 31 < kv0) continue;  // all queries precede this wave's keys
            if (qs >= a.seq) continue;
#pragma unroll
          for (int hh = 0; hh < HP; ++hh) {
            const float* lse_t = lse_all + 64 * hh;
            const float* del_t = del_all + 64 * hh;
            const int head = head0 + hh;
            // S[q][kv] and dP[q][kv]
            f32x16 s, dp;
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.f;
#pragma unroll
            for (int k = 0; k < KS; ++k) {
                const int ks = hh * KS + k;
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_kc(qt + (ks >> 2) * 8192, u * 32, ks & 3, lane), kf[ks], s, 0, 0, 0);
                dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_kc(dot + (ks >> 2) * 8192, u * 32, ks & 3, lane), vf[ks], dp, 0, 0, 0);
            }
            // P = exp2(S * c - lse[q]); dS = P * (dP - delta[q]); rows q = acc_row(r), column kv = lane.
            // Only sub-tiles on the causal diagonal or past the last query mask per element; keys
            // beyond the padding limit are whole lanes and are cleared once, after the loop.
            const bool need_mask = (a.mask == BB_MASK_CAUSAL && qs < kv0 + 31) || qs + 32 > a.seq;
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int ql = u * 32 + 8 * g4 + 4 * (lane >> 5);
                const f32x4 l4 = *(const f32x4*)(lse_t + ql);
#pragma unroll
                for (int e = 0; e < 4; ++e) s[g4 * 4 + e] = __builtin_amdgcn_exp2f(fmaf(s[g4 * 4 + e], a.scale_log2, -l4[e]));
            }
            if (need_mask) {
                asm volatile("" ::: "memory");  // a real branch: most sub-tiles skip it
                const int qlane = t * 64 + u * 32 + 4 * (lane >> 5);  // register r holds query qlane + 8*(r/4) + r%4
                const int qmin = a.mask == BB_MASK_CAUSAL ? mykv : 0;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int q = qlane + 8 * (r >> 2) + (r & 3);
                    s[r] = q >= qmin && q < a.seq ? s[r] : 0.f;
                }
            }
            // dropout: dP = dP~ o mask / (1 - p) before it meets P; P itself is masked (into what multiplied V in
            // the forward) only after dS has been formed from the unmasked probabilities
            unsigned kept = 0xffffu;
            if (DROP && a.drop.thresh) {
                asm volatile("" ::: "memory");
                const int qlane = t * 64 + u * 32 + 4 * (lane >> 5);
                kept = 0u;
                if (a.drop.small) {
                    // 32-bit indices; a query past the end is masked out above, what is decided for it does not matter
                    const uint32_t i0 = ((uint32_t)(b * a.heads + head) * (uint32_t)a.seq + (uint32_t)qlane) * (uint32_t)a.seq +
                                        (uint32_t)min(mykv, last);
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const uint32_t idx = i0 + (uint32_t)(8 * (r >> 2) + (r & 3)) * (uint32_t)a.seq;
                        const uint32_t x = bb_dropout_pair_bits32(a.drop.k0, a.drop.k1, idx >> 1);
                        const bool keep = (idx & 1) ? bb_keep_odd(x, a.drop.thresh) : bb_keep_even(x, a.drop.thresh);
                        kept |= keep ? 1u << r : 0u;
                        dp[r] = keep ? dp[r] * a.drop.scale : 0.f;
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int q = min(qlane + 8 * (r >> 2) + (r & 3), last);
                        const bool keep = bb_dropout_keep(a.drop.k0, a.drop.k1, a.drop.thresh, prob_index(a, b, head, q) + min(mykv, last));
                        kept |= keep ? 1u << r : 0u;
                        dp[r] = keep ? dp[r] * a.drop.scale : 0.f;
                    }
                }
            }
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int ql = u * 32 + 8 * g4 + 4 * (lane >> 5);
                const f32x4 d4 = *(const f32x4*)(del_t + ql);
#pragma unroll
                for (int e = 0; e < 4; ++e) dp[g4 * 4 + e] = s[g4 * 4 + e] * (dp[g4 * 4 + e] - d4[e]);
            }
            if (DROP && a.drop.thresh) {
#pragma unroll
                for (int r = 0; r < 16; ++r) s[r] = (kept >> r) & 1u ? s[r] * a.drop.scale : 0.f;
            }
            // dV^T += dO^T P~ ; dK^T += Q^T dS   (contraction over the 32 queries of this sub-tile)
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
                const bf16x8 pf = pack_acc(s, kk), dsf = pack_acc(dp, kk);
#pragma unroll
                for (int d = 0; d < DT; ++d) {
                    const int dt = hh * DT + d;
                    dv[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_tr(dot + fh * 8192, u * 32 + kk * 16, dt * 32, lane), pf, dv[dt], 0, 0, 0);
                    dk[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_tr(qt + fh * 8192, u * 32 + kk * 16, dt * 32, lane), dsf, dk[dt], 0, 0, 0);
                }
            }
          }
        }
        block_sync();
    }
    if (mykv >= pad_limit) {  // a padded key takes no probability mass: its gradients are zero
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) dk[t][r] = dv[t][r] = 0.f;
    }
    if (mykv < a.seq) {
        bf16* dkp = a.dk + (row_base + mykv) * a.ld_dqkv + hg * (64 * NPAN) + fh * 64;
        bf16* dvp = a.dv + (row_base + mykv) * a.ld_dqkv + hg * (64 * NPAN) + fh * 64;
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int d = dt * 32 + 8 * g4 + 4 * (lane >> 5);
                u32x2 wk = {pack2bf(dk[dt][g4 * 4] * a.scale, dk[dt][g4 * 4 + 1] * a.scale),
                            pack2bf(dk[dt][g4 * 4 + 2] * a.scale, dk[dt][g4 * 4 + 3] * a.scale)};
                u32x2 wv = {pack2bf(dv[dt][g4 * 4], dv[dt][g4 * 4 + 1]), pack2bf(dv[dt][g4 * 4 + 2], dv[dt][g4 * 4 + 3])};
                *(u32x2*)(dkp + d) = wk;
                *(u32x2*)(dvp + d) = wv;
            }
    }
}

// =========================================================================================
// backward dQ: block = 128 queries (4 waves x 32), loop over 64-key tiles
// =========================================================================================
template <bool DROP, int HP, int NPAN = 1>
__global__ __launch_bounds__(256, 2) void attn_bwd_dq_kernel(const AttnArgs a) {
    static_assert(HP == 1 || NPAN == 1, "pairs of heads are 32 wide");
    constexpr int KS = 4 * NPAN / HP, DT = 2 * NPAN / HP, TILE = NPAN * 8192;
    __shared__ __attribute__((aligned(16))) unsigned char smem[2 * 2 * TILE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int groups = a.heads / HP;
    const BlockMap bm = map_block(a.batch * groups);
    if (bm.bh >= a.batch * groups) return;
    const int qb = (a.seq + 127) / 128 - 1 - bm.rank;
    const int b = bm.bh / groups, hg = bm.bh % groups, head0 = hg * HP;
    const int64_t row_base = (int64_t)b * a.seq;
    const bf16* Q = a.q + row_base * a.ld_qkv + hg * (64 * NPAN);
    const bf16* K = a.k + row_base * a.ld_qkv + hg * (64 * NPAN);
    const bf16* V = a.v + row_base * a.ld_qkv + hg * (64 * NPAN);
    const bf16* DO = a.d_o + row_base * a.ld_o + hg * (64 * NPAN);
    const int q0 = qb * 128 + wave * 32;
    const int myq = q0 + (lane & 31);
    const int last = a.seq - 1;
    int kv_end = a.seq;
    if (a.mask == BB_MASK_CAUSAL) kv_end = min(a.seq, qb * 128 + 128);
    else if (a.mask == BB_MASK_KEY_PADDING) kv_end = min(a.seq, a.key_len[b]);
    const int ntiles = (kv_end + 63) / 64;
    // rows past the end compute on clamped inputs and are not stored
    const int my_limit = kv_limit(a, b, myq);
    const int wave_min_limit = kv_limit(a, b, q0);  // limits grow with the query index

    bf16x8 qf[4 * NPAN], dof[4 * NPAN];
    {
        const int64_t r = min(myq, last);
#pragma unroll
        for (int ks = 0; ks < 4 * NPAN; ++ks) {
            qf[ks] = *(const bf16x8*)(Q + r * a.ld_qkv + (lane >> 5) * 8 + ks * 16);
            dof[ks] = *(const bf16x8*)(DO + r * a.ld_o + (lane >> 5) * 8 + ks * 16);
        }
    }
    // delta[q] = rowsum(dO o O) over the head's columns: the lane and its partner (lane ^ 32) hold the two halves of
    // each 16-column step of the query's dO row; the matching halves of O are fetched once.  Written out for the
    // dK / dV kernel, which runs after this one.
    float my_lse[HP], my_delta[HP];
    {
        const bf16* O = a.o + row_base * a.ld_o + hg * (64 * NPAN);
        const int64_t r = min(myq, last);
#pragma unroll
        for (int hh = 0; hh < HP; ++hh) {
            const int64_t stat = ((int64_t)b * a.heads + head0 + hh) * a.seq + min(myq, last);
            my_lse[hh] = a.lse[stat];
            float dl = 0.f;
#pragma unroll
            for (int k = 0; k < KS; ++k) {
                const int ks = hh * KS + k;
                const bf16x8 of = *(const bf16x8*)(O + r * a.ld_o + (lane >> 5) * 8 + ks * 16);
#pragma unroll
                for (int e = 0; e < 8; ++e) dl = fmaf((float)dof[ks][e], (float)of[e], dl);
            }
            dl += __shfl_xor(dl, 32, 64);
            if (lane < 32 && myq < a.seq) a.delta[stat] = dl;
            my_delta[hh] = dl;
        }
    }
    f32x16 dq[2 * NPAN];
#pragma unroll
    for (int t = 0; t < 2 * NPAN; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) dq[t][r] = 0.f;

    const LaneOff lo = lane_off(a.ld_qkv, wave, lane);
    auto issue = [&](int t) {
        unsigned char* st = smem + (t & 1) * (2 * TILE);
        const int kv0 = t * 64;
#pragma unroll
        for (int p = 0; p < NPAN; ++p) {
            dma_tile64(K + p * 64, a.ld_qkv, kv0, last, st + p * 8192, wave, lane, lo);
            dma_tile64(V + p * 64, a.ld_qkv, kv0, last, st + TILE + p * 8192, wave, lane, lo);
        }
    };
    if (ntiles > 0) issue(0);
    for (int t = 0; t < ntiles; ++t) {
        asm volatile("" ::: "memory");
        if (t + 1 < ntiles) {
            issue(t + 1);
            wait_vm<4 * NPAN>();
        } else {
            wait_vm<0>();
        }
        block_sync();
        const unsigned char* kt = smem + (t & 1) * (2 * TILE);
        const unsigned char* vt = kt + TILE;
        const int kv0 = t * 64;
        const bool active = !(a.mask == BB_MASK_CAUSAL && kv0 > q0 + 31);
        if (active) {
#pragma unroll
            for (int u = 0; u < 2; ++u) {
#pragma unroll
              for (int hh = 0; hh < HP; ++hh) {
                const int head = head0 + hh;
                f32x16 s, dp;
#pragma unroll
                for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.f;
#pragma unroll
                for (int k = 0; k < KS; ++k) {
                    const int ks = hh * KS + k;
                    s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_kc(kt + (ks >> 2) * 8192, u * 32, ks & 3, lane), qf[ks], s, 0, 0, 0);
                    dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_kc(vt + (ks >> 2) * 8192, u * 32, ks & 3, lane), dof[ks], dp, 0, 0, 0);
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) s[r] = __builtin_amdgcn_exp2f(fmaf(s[r], a.scale_log2, -my_lse[hh]));
                if (kv0 + u * 32 + 32 > wave_min_limit) {
                    asm volatile("" ::: "memory");  // a real branch: only tiles on the mask boundary pay for it
                    const int lim = my_limit - kv0 - u * 32 - 4 * (lane >> 5);
#pragma unroll
                    for (int r = 0; r < 16; ++r) s[r] = 8 * (r >> 2) + (r & 3) < lim ? s[r] : 0.f;
                }
                if (DROP && a.drop.thresh) {
                    asm volatile("" ::: "memory");
                    const uint64_t base = prob_index(a, b, head, min(myq, last)) + kv0 + u * 32;
                    drop_acc_rows(a.drop, base, lane, dp);
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) dp[r] = s[r] * (dp[r] - my_delta[hh]);
                // dQ^T += K^T dS^T (contraction over the 32 keys of this sub-tile)
#pragma unroll
                for (int kk = 0; kk < 2; ++kk) {
                    const bf16x8 dsf = pack_acc(dp, kk);
#pragma unroll
                    for (int d = 0; d < DT; ++d) {
                        const int dt = hh * DT + d;
                        dq[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_tr(kt + (dt >> 1) * 8192, u * 32 + kk * 16, (dt & 1) * 32, lane), dsf, dq[dt], 0, 0, 0);
                    }
                }
              }
            }
        }
        block_sync();
    }
    if (myq < a.seq) {
        bf16* dqp = a.dq + (row_base + myq) * a.ld_dqkv + hg * (64 * NPAN);
#pragma unroll
        for (int dt = 0; dt < 2 * NPAN; ++dt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int d = dt * 32 + 8 * g4 + 4 * (lane >> 5);
                u32x2 w = {pack2bf(dq[dt][g4 * 4] * a.scale, dq[dt][g4 * 4 + 1] * a.scale),
                           pack2bf(dq[dt][g4 * 4 + 2] * a.scale, dq[dt][g4 * 4 + 3] * a.scale)};
                *(u32x2*)(dqp + d) = w;
            }
    }
}

// =========================================================================================
// host entry points
// =========================================================================================
static int check_attn(const char* name, int dtype, int mask, int batch, int heads, int seq, int head_dim, int64_t ld_qkv,
                      int64_t ld_o, const int32_t* key_len) {
    BB_REQUIRE(dtype == BB_BF16, "%s: the fused attention kernels are bf16 only (got dtype %d)", name, dtype);
    BB_REQUIRE(head_dim == 64 || head_dim == 128 || (head_dim == 32 && heads % 2 == 0),
               "%s: head dimension must be 64, 128, or 32 with an even number of heads (got %d, %d heads)", name, head_dim, heads);
    BB_REQUIRE(mask >= BB_MASK_NONE && mask <= BB_MASK_KEY_PADDING, "%s: bad mask %d", name, mask);
    BB_REQUIRE(mask != BB_MASK_KEY_PADDING || key_len, "%s: key_padding mask needs key_len", name);
    BB_REQUIRE(batch >= 0 && heads > 0 && seq >= 0, "%s: bad shape", name);
    BB_REQUIRE(ld_qkv % 8 == 0 && ld_o % 8 == 0 && ld_qkv >= heads * head_dim && ld_o >= heads * head_dim, "%s: bad leading dimension", name);
    BB_REQUIRE(ld_qkv < (1 << 24) && ld_o < (1 << 24), "%s: leading dimension too large", name);
    BB_REQUIRE(((int64_t)batch * heads * 2 + 8) * ((seq + 127) / 128) < (1ll << 31), "%s: batch * heads * seq exceeds the grid limit", name);
    return BB_OK;
}

extern "C" int bb_attention_fwd(int dtype, int mask, int batch, int heads, int seq, int head_dim, const void* q,
                                const void* k, const void* v, int64_t ld_qkv, void* out, int64_t ld_out, float* lse,
                                const int32_t* key_len, float dropout_p, uint32_t dropout_k0, uint32_t dropout_k1,
                                void* stream) {
    int rc = check_attn("bb_attention_fwd", dtype, mask, batch, heads, seq, head_dim, ld_qkv, ld_out, key_len);
    if (rc) return rc;
    if (batch == 0 || seq == 0) return BB_OK;
    BB_REQUIRE(q && k && v && out && lse, "bb_attention_fwd: null pointer");
    BB_REQUIRE(dropout_p >= 0.f && dropout_p < 1.f, "bb_attention_fwd: dropout_p must be in [0, 1)");
    AttnArgs a = {};
    a.drop = bb_drop_key(dropout_p, dropout_k0, dropout_k1, (uint64_t)batch * heads * (uint64_t)seq * (uint64_t)seq);
    a.q = (const bf16*)q; a.k = (const bf16*)k; a.v = (const bf16*)v;
    a.out = (bf16*)out; a.lse = lse; a.key_len = key_len;
    a.ld_qkv = ld_qkv; a.ld_o = ld_out;
    a.batch = batch; a.heads = heads; a.seq = seq; a.mask = mask;
    a.scale = 1.0f / sqrtf((float)head_dim);
    a.scale_log2 = a.scale * 1.4426950408889634f;
    // dropout is a kernel of its own: its keep decisions cost registers that decide how many blocks a CU holds
    const int hp = head_dim == 32 ? 2 : 1;   // heads per block
    const dim3 grid(attn_grid(seq, batch * (heads / hp)));
    hipStream_t st = (hipStream_t)stream;
    if (head_dim == 128) {
        if (a.drop.thresh) hipLaunchKernelGGL((attn_fwd_kernel<true, 1, 2>), grid, dim3(256), 0, st, a);
        else hipLaunchKernelGGL((attn_fwd_kernel<false, 1, 2>), grid, dim3(256), 0, st, a);
    } else if (hp == 1) {
        if (a.drop.thresh) hipLaunchKernelGGL((attn_fwd_kernel<true, 1>), grid, dim3(256), 0, st, a);
        else hipLaunchKernelGGL((attn_fwd_kernel<false, 1>), grid, dim3(256), 0, st, a);
    } else {
        if (a.drop.thresh) hipLaunchKernelGGL((attn_fwd_kernel<true, 2>), grid, dim3(256), 0, st, a);
        else hipLaunchKernelGGL((attn_fwd_kernel<false, 2>), grid, dim3(256), 0, st, a);
    }
    BB_LAUNCH_CHECK();
    return BB_OK;
}

extern "C" int bb_attention_bwd(int dtype, int mask, int batch, int heads, int seq, int head_dim, const void* q,
                                const void* k, const void* v, int64_t ld_qkv, const void* out, const void* d_out,
                                int64_t ld_out, const float* lse, float* delta, void* dq, void* dk, void* dv,
                                int64_t ld_dqkv, const int32_t* key_len, float dropout_p, uint32_t dropout_k0,
                                uint32_t dropout_k1, void* stream) {
    int rc = check_attn("bb_attention_bwd", dtype, mask, batch, heads, seq, head_dim, ld_qkv, ld_out, key_len);
    if (rc) return rc;
    if (batch == 0 || seq == 0) return BB_OK;
    BB_REQUIRE(q && k && v && out && d_out && lse && delta && dq && dk && dv, "bb_attention_bwd: null pointer");
    BB_REQUIRE(ld_dqkv % 4 == 0 && ld_dqkv >= heads * head_dim, "bb_attention_bwd: bad gradient leading dimension");
    BB_REQUIRE(dropout_p >= 0.f && dropout_p < 1.f, "bb_attention_bwd: dropout_p must be in [0, 1)");
    AttnArgs a = {};
    a.drop = bb_drop_key(dropout_p, dropout_k0, dropout_k1, (uint64_t)batch * heads * (uint64_t)seq * (uint64_t)seq);
    a.q = (const bf16*)q; a.k = (const bf16*)k; a.v = (const bf16*)v;
    a.o = (const bf16*)out; a.d_o = (const bf16*)d_out;
    a.dq = (bf16*)dq; a.dk = (bf16*)dk; a.dv = (bf16*)dv;
    a.lse = (float*)lse; a.delta = delta; a.key_len = key_len;
    a.ld_qkv = ld_qkv; a.ld_o = ld_out; a.ld_dqkv = ld_dqkv;
    a.batch = batch; a.heads = heads; a.seq = seq; a.mask = mask;
    a.scale = 1.0f / sqrtf((float)head_dim);
    a.scale_log2 = a.scale * 1.4426950408889634f;
    hipStream_t st = (hipStream_t)stream;
    // the dQ kernel first: it also leaves delta = rowsum(dO o O) of its queries for the dK / dV kernel
    const int hp = head_dim == 32 ? 2 : 1;   // heads per block
    dim3 grid(attn_grid(seq, batch * (heads / hp)));
    if (head_dim == 128) {
        // two dK / dV blocks per head and key block (one per 64-wide half of the columns), their LDS from the launch
        constexpr int smem = 2 * (2 * 2 * 8192 + 512);
        const dim3 grid2(attn_grid(seq, batch * heads * 2));
        if (a.drop.thresh) {
            BB_HIP_CHECK(bb_allow_dynamic_lds((const void*)attn_bwd_dkv_kernel<true, 1, 2>, smem));
            hipLaunchKernelGGL((attn_bwd_dq_kernel<true, 1, 2>), grid, dim3(256), 0, st, a);
            hipLaunchKernelGGL((attn_bwd_dkv_kernel<true, 1, 2>), grid2, dim3(256), smem, st, a);
        } else {
            BB_HIP_CHECK(bb_allow_dynamic_lds((const void*)attn_bwd_dkv_kernel<false, 1, 2>, smem));
            hipLaunchKernelGGL((attn_bwd_dq_kernel<false, 1, 2>), grid, dim3(256), 0, st, a);
            hipLaunchKernelGGL((attn_bwd_dkv_kernel<false, 1, 2>), grid2, dim3(256), smem, st, a);
        }
    } else if (hp == 1) {
        if (a.drop.thresh) {
            hipLaunchKernelGGL((attn_bwd_dq_kernel<true, 1>), grid, dim3(256), 0, st, a);
            hipLaunchKernelGGL((attn_bwd_dkv_kernel<true, 1>), grid, dim3(256), 0, st, a);
        } else {
            hipLaunchKernelGGL((attn_bwd_dq_kernel<false, 1>), grid, dim3(256), 0, st, a);
            hipLaunchKernelGGL((attn_bwd_dkv_kernel<false, 1>), grid, dim3(256), 0, st, a);
        }
    } else {
        if (a.drop.thresh) {
            hipLaunchKernelGGL((attn_bwd_dq_kernel<true, 2>), grid, dim3(256), 0, st, a);
            hipLaunchKernelGGL((attn_bwd_dkv_kernel<true, 2>), grid, dim3(256), 0, st, a);
        } else {
            hipLaunchKernelGGL((attn_bwd_dq_kernel<false, 2>), grid, dim3(256), 0, st, a);
            hipLaunchKernelGGL((attn_bwd_dkv_kernel<false, 2>), grid, dim3(256), 0, st, a);
        }
    }
    BB_LAUNCH_CHECK();
    return BB_OK;
}
