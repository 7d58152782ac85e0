// MFMA GEMM for gfx950: bf16 (v_mfma_f32_32x32x16_bf16) and fp32 (v_mfma_f32_32x32x2_f32),
// LDS-tiled, double-buffered, batched with two-level strides, fused epilogues.
//
// Stands in for F.linear / torch.matmul and their autograd backward in the reference layer
// (DeepSpeedExamples/pipeline_parallelism/transformer.py:121,127,136-146,158).
//
// bf16 data path.  Both operand tiles are kept in LDS "k-contiguous": tile row r (an m- or
// n-index) owns 64 consecutive k values = 8 chunks of 16 bytes, chunk c stored at chunk slot
// c ^ swz(r) so that the 16-byte fragment reads of 16 consecutive rows hit distinct banks.
// An operand whose memory layout is k-major (the transposed operand of NN / TN) is loaded as
// 16-byte vectors along its contiguous dimension and transposed in registers before the LDS
// store, so the MFMA side never changes.
#include "gemm_kernels.h"

// =========================================================================================
// host dispatch
// =========================================================================================
template <int BM, int BN, int WM, int WN, bool TA, bool TB>
static int launch_bf16(GemmArgs& g, int batches, hipStream_t st) {
    constexpr int smem = 2 * (BM + BN) * 64 * 2;
    auto kern = gemm_bf16_kernel<BM, BN, WM, WN, TA, TB>;
    BB_HIP_CHECK(bb_allow_dynamic_lds((const void*)kern, smem));
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    dim3 grid(g.tiles_m * g.tiles_n, 1, batches);
    hipLaunchKernelGGL(kern, grid, dim3(WM * WN * 64), smem, st, g);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

// Tile choice: the largest tile that still gives every CU work; small problems (attention
// heads: 64-wide operands) take the 128x64 / 64x128 tiles.
enum Bf16Tile { T128x64 = 0, T64x128, T256x256, T256x128, T128x128 };
static const char* const kBf16TileNames[] = {"128x64", "64x128", "256x256", "256x128", "128x128"};

static Bf16Tile pick_bf16_tile(int M, int N, int64_t batches) {
    const int64_t t2128 = (int64_t)((M + 255) / 256) * ((N + 127) / 128) * batches;
    if (N <= 64) return T128x64;
    if (M <= 64) return T64x128;
    if (M >= 256 && N >= 128 && t2128 >= 200) return T256x128;
    return T128x128;
}

template <int BM, int BN, int WM, int WN, bool AKM, bool BKM, bool DB, int STAGES = 4, int BK = 32>
static int launch_bf16_dma(GemmArgs& g, int batches, hipStream_t st) {
    constexpr int smem = STAGES * (BM + BN) * BK * 2;
    auto kern = gemm_bf16_dma_kernel<BM, BN, WM, WN, AKM, BKM, DB, STAGES, BK>;
    if constexpr (!AKM && !BKM) {       // dropout goes with forward (NT) products only: fill_args refuses the others
        if (g.drop.thresh) kern = gemm_bf16_dma_kernel<BM, BN, WM, WN, AKM, BKM, DB, STAGES, BK, true>;
    }
    BB_HIP_CHECK(bb_allow_dynamic_lds((const void*)kern, smem));
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    dim3 grid(g.tiles_m * g.tiles_n, 1, batches);
    hipLaunchKernelGGL(kern, grid, dim3(WM * WN * 64), smem, st, g);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

// persistent kernels: one block per CU walks the tiles
static constexpr int kPersistBlocks = 256;
template <int BM, int BN, int WM, int WN, bool TB> static int launch_bf16_dma_persist(GemmArgs& g, hipStream_t st) {
    constexpr int smem = 3 * (BM + BN) * 32 * 2 + WM * WN * 32 * 64 * 4;
    auto kern = gemm_bf16_dma_persist_kernel<BM, BN, WM, WN, TB, false>;
    if constexpr (!TB) {
        if (g.drop.thresh) kern = gemm_bf16_dma_persist_kernel<BM, BN, WM, WN, TB, true>;
    }
    BB_HIP_CHECK(bb_allow_dynamic_lds((const void*)kern, smem));
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    const int total = g.tiles_m * g.tiles_n;
    hipLaunchKernelGGL(kern, dim3(total < kPersistBlocks ? (total + 7) / 8 * 8 : kPersistBlocks), dim3(WM * WN * 64), smem, st, g);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

template <int BM, int BN, int WM, int WN>
static int launch_bf16_dma_stats(GemmArgs& g, hipStream_t st) {
    constexpr int smem = 3 * (BM + BN) * 64 * 2;
    auto kern = gemm_bf16_dma_stats_kernel<BM, BN, WM, WN>;
    BB_HIP_CHECK(bb_allow_dynamic_lds((const void*)kern, smem));
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(WM * WN * 64), smem, st, g);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

template <int BM, int BN, int WM, int WN>
static int launch_bf16_dma_bnbwd(GemmArgs& g, const BnBwdArgs& bn, hipStream_t st) {
    constexpr int smem = 3 * (BM + BN) * 64 * 2;
    auto kern = gemm_bf16_dma_bnbwd_kernel<BM, BN, WM, WN>;
    BB_HIP_CHECK(bb_allow_dynamic_lds((const void*)kern, smem));
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(WM * WN * 64), smem, st, g, bn);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

// DMA kernels need K % 32 == 0 and at least one full vector of rows; tile by problem size
enum DmaTile { D_NONE = 0, D256x256w8db, D256x128w8db, D128x128s3, D256x256k64, D256x128k64s3, D128x128k64, D128x64k64s3, D128x64s3,
               D64x128k64s3, D64x128s3, D256x192k64, D256x256p };
static const char* const kDmaTileNames[] = {"", "dma256x256w8db", "dma256x128w8db", "dma128x128s3", "dma256x256k64", "dma256x128k64s3",
                                            "dma128x128k64", "dma128x64k64s3", "dma128x64s3", "dma64x128k64s3", "dma64x128s3",
                                            "dma256x192k64", "dma256x256p"};
// The tile of a problem depends on its shape, layout and epilogue kind only (never on the stream, the environment or
// what ran before), and every kernel adds up a contraction in the same order: a redundant forward and a normal forward
// of the same layer give the same bits.
static DmaTile pick_dma_tile(int M, int N, int K, int64_t batches, int layout) {
    if (K % 32 != 0 || K < 64 || M < 128 || N < 128 || N % 8 != 0) return D_NONE;
    // Rules read off sweeps of M 2048..16384 x N 768..6400 x K 1024/4096 (NT and NN) on MI355X (256 CUs,
    // one block of the 256-row tiles per CU).
    //  - Operands whose rows are k-contiguous (both of NT, A of NN) load faster as 64-wide k-tiles: one
    //    DMA instruction then covers 8 whole 128-byte lines instead of 16 half lines.  The smaller the
    //    tile, the more of its time is loading and the more that buys (128x128: up to +19 %, 256x128:
    //    +3..8 %, 256x256: +4 % at long K, and +2 % on the whole stage with the K = 1024 FFN product on it).
    //  - Above one round of 256x256 tiles they win while the last round is well filled; otherwise the
    //    small tiles, several blocks per CU, smooth the tail.  Where the sweep (outputs that stay in the
    //    last-level cache) and the stage itself (outputs that go to HBM) disagree, the stage decides: it
    //    wants the 256x256 tile from a 70 % full last round on for NT, and three stages for every 256x128
    //    problem.
    //  - Within one round: 256x256 once 256x128 tiles would need a second round, 256x128 from about half
    //    a round on, and 128x128 tiles for anything smaller.
    const bool nt = layout == BB_NT, nn = layout == BB_NN;
    const bool k64 = (nt || nn) && K % 64 == 0 && K >= 128;
    const DmaTile small = k64 && (nt || K >= 2048) ? D128x128k64 : D128x128s3;
    const DmaTile mid = !k64 ? D256x128w8db : D256x128k64s3;
    const int64_t t256 = (int64_t)((M + 255) / 256) * ((N + 255) / 256) * batches;
    const int64_t t2128 = (int64_t)((M + 255) / 256) * ((N + 127) / 128) * batches;
    const int64_t t128 = (int64_t)((M + 127) / 128) * ((N + 127) / 128) * batches;
    const bool big_ok = M >= 256 && N >= 256;
    //  - Problems with so few 128x128 tiles that half the CUs would idle (the 256-channel convolutions of a
    //    ResNet stage: 98 tiles) take 128x64 tiles: twice the blocks.
    //    (a k-major operand needs 128 rows for its swizzle, so NT narrows N and NN narrows M; TN keeps
    //    128x128).
    //  - A short forward contraction (K <= 512: the 1x1 convolution out of 256 channels) leaves a launch that is mostly
    //    its epilogue: 128x64 tiles, so that every CU stores a share (6272x1024x256: 15 us on 100 tiles of 256x128,
    //    13 us on 784 of 128x64; the input gradient of the same shape gains nothing from 64x128 tiles).
    if (K <= 512 && nt) return k64 ? D128x64k64s3 : D128x64s3;
    if (t128 <= 128 && nt) return k64 ? D128x64k64s3 : D128x64s3;
    if (t128 <= 128 && nn) return k64 ? D64x128k64s3 : D64x128s3;
    //  - NT problems whose 256x256 tiles would fill under 70 % of their rounds may take 256x192 tiles (six
    //    accumulator tiles per wave, about 9 % below the 256x256 tile at equal fill) instead of falling back
    //    to 128x128: compared by the share of the occupied tile slots that is real output.  (Alone, the QKV
    //    projection 8192x3072 - 1.5 rounds of 256x256 tiles, exactly two of 256x192 - is 19 % faster on them;
    //    inside the power-limited stage the whole batch is 1 % slower, so 75 % full rounds stay on 256x256.)
    if (nt && k64 && big_ok && t2128 > 256) {
        auto useful = [&](int bn) {   // real output / output slots of whole rounds
            const int64_t t = (int64_t)((M + 255) / 256) * ((N + bn - 1) / bn) * batches;
            return (double)M * N * batches / ((double)((t + 255) / 256 * 256) * 256 * bn);
        };
        const double s256 = useful(256), s192 = 0.91 * useful(192);
        if (s256 < 0.70 && s192 > s256 && s192 >= 0.65) return D256x192k64;
    }
    if (t256 > 256) {
        const int64_t slots = (t256 + 255) / 256 * 256;
        const bool full85 = t256 * 100 >= slots * 85, full70 = t256 * 10 >= slots * 7;
        if (!big_ok) return small;
        if (k64 && nt) {
            // a last round under 85 %: 256x128 tiles if those come out in whole rounds (the QKV projection
            // 8192x3072: 1.5 rounds of 256x256, exactly three of 256x128; +1 % on the stage)
            const int64_t slots2 = (t2128 + 255) / 256 * 256;
            if (full85) return D256x256k64;
            if (t2128 * 10 >= slots2 * 9) return mid;
            return full70 ? D256x256k64 : small;
        }
        if (k64) return full85 || (K >= 2048 && full70) ? D256x256w8db : small;
        return full70 || K >= 1536 ? D256x256w8db : small;
    }
    if (big_ok && t2128 > 256) return k64 && nt ? D256x256k64 : D256x256w8db;
    if (M >= 256 && t2128 > 136) return mid;
    return small;
}

// The tile of a (shape, layout, epilogue kind): NT / NN problems of more than one round of 256x256 tiles take the
// persistent kernel (blocks walk their tiles with the DMA ring running through the tile boundaries) unless the epilogue
// evaluates the activation: that work keeps the vector ALUs busy for about as long as the tile's matrix work does, the
// boundary is not what such a launch waits for (FFN1 with act + act': 114 us on the plain kernel, 118 persistent;
// the plain product 95 against 77).  All kernels add up a contraction in the same order: which one runs changes no bit.
static DmaTile pick_dma_tile_for(int M, int N, int K, int64_t batches, int layout, int epilogue) {
    const DmaTile t = pick_dma_tile(M, N, K, batches, layout);
    const bool light = epilogue != BB_EPI_ACT && epilogue != BB_EPI_ACT_DACT && epilogue != BB_EPI_DACT;
    const int64_t t256 = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
    if ((t == D256x256k64 || t == D256x256w8db) && light && batches == 1 && layout != BB_TN && K % 64 == 0 && t256 > kPersistBlocks)
        return D256x256p;
    return t;
}

template <bool TA, bool TB> static int dispatch_bf16(GemmArgs& g, int batches, hipStream_t st) {
    switch (pick_dma_tile_for(g.M, g.N, g.K, batches, TA ? BB_TN : TB ? BB_NN : BB_NT, g.epilogue)) {
        case D256x256w8db: return launch_bf16_dma<256, 256, 2, 4, TA, TB, true>(g, batches, st);
        case D256x128w8db: return launch_bf16_dma<256, 128, 4, 2, TA, TB, true>(g, batches, st);
        case D128x128s3: return launch_bf16_dma<128, 128, 2, 2, TA, TB, true, 3>(g, batches, st);
        case D256x256k64: return launch_bf16_dma<256, 256, 2, 4, TA, TB, true, 2, 64>(g, batches, st);
        case D256x128k64s3: return launch_bf16_dma<256, 128, 4, 2, TA, TB, true, 3, 64>(g, batches, st);
        case D128x128k64: return launch_bf16_dma<128, 128, 2, 2, TA, TB, true, 2, 64>(g, batches, st);
        case D128x64k64s3: return launch_bf16_dma<128, 64, 4, 1, TA, TB, true, 3, 64>(g, batches, st);
        case D128x64s3: return launch_bf16_dma<128, 64, 4, 1, TA, TB, true, 3>(g, batches, st);
        case D64x128k64s3: return launch_bf16_dma<64, 128, 2, 2, TA, TB, true, 3, 64>(g, batches, st);
        case D64x128s3: return launch_bf16_dma<64, 128, 2, 2, TA, TB, true, 3>(g, batches, st);
        case D256x256p:
            if constexpr (!TA) return launch_bf16_dma_persist<256, 256, 2, 4, TB>(g, st);
            else break;
        case D256x192k64:
            // k-contiguous operands only (192 rows do not divide into the k-major loader's instructions)
            if constexpr (!TA && !TB) return launch_bf16_dma<256, 192, 4, 2, TA, TB, true, 2, 64>(g, batches, st);
            else break;
        default: break;
    }
    switch (pick_bf16_tile(g.M, g.N, batches)) {
        case T128x64: return launch_bf16<128, 64, 4, 1, TA, TB>(g, batches, st);
        case T64x128: return launch_bf16<64, 128, 1, 4, TA, TB>(g, batches, st);
        case T256x128: return launch_bf16<256, 128, 4, 2, TA, TB>(g, batches, st);
        default: return launch_bf16<128, 128, 2, 2, TA, TB>(g, batches, st);
    }
}

static int pick_f32_tile(int M, int N, int64_t batches) {
    const int64_t t128 = (int64_t)((M + 127) / 128) * ((N + 127) / 128) * batches;
    return t128 < 2 * 256 ? 64 : 128;
}
// Problems with fewer than two 64x64 tiles per CU (one or two waves per SIMD, and some CUs with twice the tiles of
// others) and at least 32 k-tiles wait for operands most of the time: they take 64x32 tiles whose contraction two
// groups of two waves share (kF32SplitGroups; twice the tiles, each wave's chain of k-tiles halved).  NT and NN only:
// the weight gradients (TN) of a layer share a grouped launch.
static constexpr int kF32SplitGroups = 2, kF32SplitBN = 32;
static bool pick_f32_split(int M, int N, int K, int64_t batches, int layout) {
    if (layout == BB_TN || pick_f32_tile(M, N, batches) != 64) return false;
    const int64_t t64 = (int64_t)((M + 63) / 64) * ((N + 63) / 64) * batches;
    return t64 < 2 * 256 && K >= 512;
}
template <bool TA, bool TB> static int dispatch_f32(GemmArgs& g, int batches, hipStream_t st) {
    // 64x64 tiles while 128x128 ones would leave most CUs with a single block (one wave per SIMD): shape only, and the
    // same order of additions on both, so which one runs changes no bit
    const int tile = pick_f32_tile(g.M, g.N, batches);
    g.tiles_m = (g.M + tile - 1) / tile;
    g.tiles_n = (g.N + tile - 1) / tile;
    dim3 grid(g.tiles_m * g.tiles_n, 1, batches);
    if (pick_f32_split(g.M, g.N, g.K, batches, TA ? BB_TN : TB ? BB_NN : BB_NT)) {
        g.tiles_n = (g.N + kF32SplitBN - 1) / kF32SplitBN;
        grid.x = g.tiles_m * g.tiles_n;
        hipLaunchKernelGGL((gemm_f32_ksplit_kernel<TA, TB, kF32SplitGroups, kF32SplitBN>), grid, dim3(4 * kF32SplitBN * kF32SplitGroups), 0, st, g);
    }
    else if (tile == 64) hipLaunchKernelGGL((gemm_f32_kernel<TA, TB, 64>), grid, dim3(256), 0, st, g);
    else hipLaunchKernelGGL((gemm_f32_kernel<TA, TB, 128>), grid, dim3(256), 0, st, g);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

extern "C" int bb_gemm_variant(const bb_gemm_desc* d, char* out, int out_len) {
    BB_REQUIRE(d && out && out_len > 0, "bb_gemm_variant: bad arguments");
    static const char* const layouts[] = {"nt", "nn", "tn"};
    BB_REQUIRE(d->layout >= BB_NT && d->layout <= BB_TN, "bb_gemm_variant: bad layout %d", d->layout);
    const int64_t batches = (int64_t)(d->nb1 > 0 ? d->nb1 : 1) * (d->nb2 > 0 ? d->nb2 : 1);
    if (d->dtype == BB_BF16) {
        const DmaTile dt = pick_dma_tile_for(d->M, d->N, d->K, batches, d->layout, d->epilogue);
        snprintf(out, out_len, "bf16_%s_%s", layouts[d->layout],
                 dt != D_NONE ? kDmaTileNames[dt] : kBf16TileNames[pick_bf16_tile(d->M, d->N, batches)]);
    }
    else
    {
        const int tile = pick_f32_tile(d->M, d->N, batches);
        if (pick_f32_split(d->M, d->N, d->K, batches, d->layout))
            snprintf(out, out_len, "f32_%s_64x%dk%d", layouts[d->layout], kF32SplitBN, kF32SplitGroups);
        else snprintf(out, out_len, "f32_%s_%dx%d", layouts[d->layout], tile, tile);
    }
    return BB_OK;
}

static int fill_args(const bb_gemm_desc* d, GemmArgs& g, int64_t& batches, bool& ta, bool& tb) {
    BB_REQUIRE(d != nullptr, "bb_gemm: null descriptor");
    BB_REQUIRE(d->dtype == BB_F32 || d->dtype == BB_BF16, "bb_gemm: bad dtype %d", d->dtype);
    BB_REQUIRE(d->c_dtype == d->dtype || d->c_dtype == BB_F32, "bb_gemm: bad c_dtype %d", d->c_dtype);
    BB_REQUIRE(d->layout >= BB_NT && d->layout <= BB_TN, "bb_gemm: bad layout %d", d->layout);
    BB_REQUIRE(d->M >= 0 && d->N >= 0 && d->K >= 0, "bb_gemm: negative dimension");
    BB_REQUIRE(!d->accumulate || d->c_dtype == BB_F32, "bb_gemm: accumulate needs an fp32 C");
    BB_REQUIRE(d->epilogue >= BB_EPI_NONE && d->epilogue <= BB_EPI_MUL_POS, "bb_gemm: bad epilogue");
    const int nb1 = d->nb1 > 0 ? d->nb1 : 1, nb2 = d->nb2 > 0 ? d->nb2 : 1;
    batches = (int64_t)nb1 * nb2;
    ta = d->layout == BB_TN;
    tb = d->layout != BB_NT;
    g.M = d->M; g.N = d->N; g.K = d->K; g.nb2 = nb2;
    if (d->M == 0 || d->N == 0) return BB_OK;
    BB_REQUIRE(d->A && d->B && d->C, "bb_gemm: null operand");
    BB_REQUIRE((d->epilogue != BB_EPI_DACT && d->epilogue != BB_EPI_MUL && d->epilogue != BB_EPI_MUL_POS && d->epilogue != BB_EPI_MUL_POS) || d->aux_in,
               "bb_gemm: DACT / MUL / MUL_POS epilogue needs aux_in");
    BB_REQUIRE(d->epilogue != BB_EPI_RESIDUAL || d->resid, "bb_gemm: RESIDUAL epilogue needs resid");
    BB_REQUIRE(d->epilogue != BB_EPI_ACT_DACT || d->aux_out, "bb_gemm: ACT_DACT epilogue needs aux_out");
    BB_REQUIRE(batches <= 65535, "bb_gemm: too many batches (%lld)", (long long)batches);
    const int vec = d->dtype == BB_BF16 ? 8 : 4;
    const bool conv = d->conv_c != 0 || d->conv_h != 0 || d->conv_w != 0 || d->conv_row0 != 0;
    if (conv) {
        // B = patch matrix of an NHWC tensor, gathered by the grouped DMA kernel's loader
        BB_REQUIRE(d->layout == BB_TN && d->dtype == BB_BF16 && batches == 1, "bb_gemm: a patch-matrix B needs BB_TN, bf16, no batching");
        BB_REQUIRE(d->conv_c > 0 && d->conv_c % 128 == 0 && d->conv_h > 0 && d->conv_w > 0 && d->conv_row0 >= 0,
                   "bb_gemm: patch-matrix B: conv_c (%d) must be a positive multiple of 128, conv_h/conv_w positive", d->conv_c);
        BB_REQUIRE(d->N == 9 * d->conv_c, "bb_gemm: patch-matrix B: N (%d) must be 9 * conv_c (%d)", d->N, d->conv_c);
        BB_REQUIRE(d->K % 32 == 0 && d->K >= 64 && d->M >= 128 && 32 / d->conv_w + 1 <= d->conv_h,
                   "bb_gemm: patch-matrix B: K (%d) must be a multiple of 32 and >= 64, M (%d) >= 128, and 32 pixels must "
                   "not span more than one image boundary (%d x %d)", d->K, d->M, d->conv_h, d->conv_w);
        BB_REQUIRE(!d->bias && d->epilogue == BB_EPI_NONE, "bb_gemm: patch-matrix B takes no bias / epilogue");
    }
    // the contiguous dimension of every operand is read in 16-byte vectors
    const int a_contig = ta ? d->M : d->K, b_contig = conv ? d->conv_c : tb ? d->N : d->K;
    const int64_t ldb = conv ? d->conv_c : d->ldb;
    BB_REQUIRE(a_contig % vec == 0 && d->lda % vec == 0, "bb_gemm: A contiguous dim/lda must be a multiple of %d", vec);
    BB_REQUIRE(b_contig % vec == 0 && ldb % vec == 0, "bb_gemm: B contiguous dim/ldb must be a multiple of %d", vec);
    BB_REQUIRE(((uintptr_t)d->A % 16) == 0 && ((uintptr_t)d->B % 16) == 0, "bb_gemm: operands must be 16-byte aligned");
    BB_REQUIRE(d->sA1 % vec == 0 && d->sA2 % vec == 0 && d->sB1 % vec == 0 && d->sB2 % vec == 0,
               "bb_gemm: batch strides of A/B must be multiples of %d", vec);
    BB_REQUIRE(d->lda >= a_contig && ldb >= b_contig && d->ldc >= d->N, "bb_gemm: leading dimension too small");
    g.A = d->A; g.B = d->B; g.C = d->C;
    g.bias = d->bias; g.aux_in = d->aux_in; g.aux_out = d->aux_out; g.resid = d->resid;
    g.colsum = nullptr;
    BB_REQUIRE(!d->colsum_out || d->layout == BB_TN, "bb_gemm: colsum_out needs the BB_TN layout");
    g.lda = d->lda; g.ldb = ldb; g.ldc = d->ldc; g.ldaux = d->ldaux > 0 ? d->ldaux : d->ldc;
    g.conv_h = d->conv_h; g.conv_w = d->conv_w; g.conv_c = d->conv_c; g.conv_row0 = d->conv_row0;
    g.strip_stats = nullptr;   // bb_gemm sets it where the kernel that runs the problem produces them
    g.sA1 = d->sA1; g.sA2 = d->sA2; g.sB1 = d->sB1; g.sB2 = d->sB2; g.sC1 = d->sC1; g.sC2 = d->sC2;
    g.alpha = d->alpha;
    g.epilogue = d->epilogue; g.act = d->act; g.accumulate = d->accumulate;
    g.c_f32 = (d->c_dtype == BB_F32);
    BB_REQUIRE(d->dropout_p >= 0.f && d->dropout_p < 1.f, "bb_gemm: dropout_p must be in [0, 1)");
    BB_REQUIRE(d->dropout_p == 0.f || (batches == 1 && d->layout == BB_NT && d->epilogue != BB_EPI_DACT && d->epilogue != BB_EPI_MUL && d->epilogue != BB_EPI_MUL_POS &&
                                       !d->accumulate),
               "bb_gemm: dropout goes with an unbatched, non-accumulating NT problem and not with the DACT / MUL / MUL_POS epilogues");
    g.drop = bb_drop_key(d->dropout_p, d->dropout_k0, d->dropout_k1, (uint64_t)d->M * (uint64_t)d->N);
    g.tiles_m = g.tiles_n = 0;
    return BB_OK;
}

// The bias-gradient column sums ride inside the DMA kernel when it runs the problem; otherwise
// the stand-alone reduction computes them.
static bool colsum_fusable(const bb_gemm_desc* d, int64_t batches) {
    return d->colsum_out && d->dtype == BB_BF16 && batches == 1 && pick_dma_tile(d->M, d->N, d->K, 1, d->layout) != D_NONE;
}
static int colsum_standalone(const bb_gemm_desc* d, void* stream) {
    BB_REQUIRE(d->colsum_ws, "bb_gemm: colsum_out on this problem needs colsum_ws");
    return bb_colsum_acc(d->dtype, d->K, d->M, d->A, d->lda, d->colsum_out, d->colsum_ws, stream);
}

extern "C" int bb_gemm_strip_stats_supported(const bb_gemm_desc* d) {
    return d && d->dtype == BB_BF16 && d->c_dtype == BB_BF16 && d->layout == BB_NT && d->nb1 <= 1 && d->nb2 <= 1 &&
           d->M >= 128 && d->N >= 64 && d->N % 8 == 0 && d->K >= 128 && d->K % 64 == 0 && d->conv_c == 0 && !d->colsum_out &&
           !d->bias && d->epilogue == BB_EPI_NONE && d->alpha == 1.0f && d->dropout_p == 0.f;
}
extern "C" int64_t bb_strip_stats_workspace(int rows, int cols) { return (int64_t)((rows + 31) / 32) * 3 * cols; }

extern "C" int64_t bb_bn_bwd_strips_workspace(int rows, int cols) { return (int64_t)((rows + 31) / 32) * 2 * cols; }

static int check_bn_bwd_stats(const char* name, const bb_bn_bwd_stats* bn) {
    BB_REQUIRE(bn && bn->x && bn->mean && bn->rstd && bn->strips, "%s: null pointer in bb_bn_bwd_stats", name);
    BB_REQUIRE(((uintptr_t)bn->x % 16) == 0 && ((uintptr_t)bn->mean % 16) == 0 && ((uintptr_t)bn->rstd % 16) == 0 &&
               ((uintptr_t)bn->strips % 16) == 0, "%s: the bb_bn_bwd_stats operands must be 16-byte aligned", name);
    return BB_OK;
}

extern "C" int bb_gemm_bn_bwd_supported(const bb_gemm_desc* d) {
    return d && d->dtype == BB_BF16 && d->c_dtype == BB_BF16 && d->layout == BB_NN && d->nb1 <= 1 && d->nb2 <= 1 &&
           d->M >= 128 && d->N >= 128 && d->N % 8 == 0 && d->K >= 128 && d->K % 64 == 0 && d->conv_c == 0 && !d->colsum_out &&
           !d->strip_stats && !d->bias && !d->accumulate && d->alpha == 1.0f && d->dropout_p == 0.f && d->ldc == d->N &&
           (d->ldaux == 0 || d->ldaux == d->N) &&
           (d->epilogue == BB_EPI_NONE || (d->epilogue == BB_EPI_RESIDUAL && d->resid) || (d->epilogue == BB_EPI_MUL_POS && d->aux_in));
}

extern "C" int bb_gemm_bn_bwd(const bb_gemm_desc* d, const bb_bn_bwd_stats* bn, void* stream) {
    BB_REQUIRE(bb_gemm_bn_bwd_supported(d), "bb_gemm_bn_bwd: needs an unbatched bf16 BB_NN problem with a contiguous bf16 C, M >= 128, "
               "N >= 128, N %% 8 == 0, K >= 128, K %% 64 == 0, alpha = 1, no bias, epilogue BB_EPI_NONE, BB_EPI_RESIDUAL or BB_EPI_MUL_POS");
    int rc = check_bn_bwd_stats("bb_gemm_bn_bwd", bn);
    if (rc) return rc;
    GemmArgs g;
    int64_t batches;
    bool ta, tb;
    rc = fill_args(d, g, batches, ta, tb);
    if (rc) return rc;
    const BnBwdArgs b = {bn->x, bn->mean, bn->rstd, bn->strips};
    // the tile the plain product of this shape would take, where it is one of the two built with the sums
    if (pick_dma_tile(d->M, d->N, d->K, 1, BB_NN) == D256x128k64s3) return launch_bf16_dma_bnbwd<256, 128, 4, 2>(g, b, (hipStream_t)stream);
    return launch_bf16_dma_bnbwd<64, 128, 2, 2>(g, b, (hipStream_t)stream);
}

extern "C" int bb_gemm(const bb_gemm_desc* d, void* stream) {
    if (d && d->conv_c != 0) return bb_gemm_grouped(d, 1, stream);   // only the grouped kernel gathers a patch-matrix B
    if (d && d->strip_stats) {
        BB_REQUIRE(bb_gemm_strip_stats_supported(d), "bb_gemm: strip_stats needs an unbatched bf16 BB_NT problem with a bf16 C, "
                   "M >= 128, N >= 64, N %% 8 == 0, K >= 128, K %% 64 == 0, alpha = 1, no bias, no epilogue");
        BB_REQUIRE(((uintptr_t)d->strip_stats % 16) == 0, "bb_gemm: strip_stats must be 16-byte aligned");
        GemmArgs g;
        int64_t batches;
        bool ta, tb;
        int rc = fill_args(d, g, batches, ta, tb);
        if (rc) return rc;
        g.strip_stats = d->strip_stats;
        // the two tiles that carry the statistics: 256x128 where the ordinary choice would be that tile, else 128x64
        if (pick_dma_tile(d->M, d->N, d->K, 1, BB_NT) == D256x128k64s3) return launch_bf16_dma_stats<256, 128, 4, 2>(g, (hipStream_t)stream);
        return launch_bf16_dma_stats<128, 64, 4, 1>(g, (hipStream_t)stream);
    }
    GemmArgs g;
    int64_t batches;
    bool ta, tb;
    int rc = fill_args(d, g, batches, ta, tb);
    if (rc) return rc;
    if (d->M == 0 || d->N == 0) return BB_OK;
    hipStream_t st = (hipStream_t)stream;
    if (d->colsum_out) {
        if (colsum_fusable(d, batches)) g.colsum = d->colsum_out;
        else if ((rc = colsum_standalone(d, stream)) != BB_OK) return rc;
    }
    if (d->dtype == BB_BF16) {
        if (!ta && !tb) return dispatch_bf16<false, false>(g, (int)batches, st);
        if (!ta && tb) return dispatch_bf16<false, true>(g, (int)batches, st);
        return dispatch_bf16<true, true>(g, (int)batches, st);
    }
    if (!ta && !tb) return dispatch_f32<false, false>(g, (int)batches, st);
    if (!ta && tb) return dispatch_f32<false, true>(g, (int)batches, st);
    return dispatch_f32<true, true>(g, (int)batches, st);
}

template <int BM, int BN, int WM, int WN, bool BKM, int STAGES, bool STATS = false>
static int launch_conv3x3(GemmArgs& g, const ConvArgs& cv, hipStream_t st) {
    constexpr int smem = STAGES * (BM + BN) * 64 * 2;
    auto kern = conv3x3_bf16_igemm_kernel<BM, BN, WM, WN, BKM, STAGES, STATS>;
    BB_HIP_CHECK(bb_allow_dynamic_lds((const void*)kern, smem));
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(WM * WN * 64), smem, st, g, cv);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

extern "C" int bb_conv3x3_supported(int dtype, int mode, int n, int h, int w, int cin, int cout) {
    const int64_t rows = (int64_t)n * h * w;
    const int gathered = mode == BB_CONV_DGRAD ? cout : cin, produced = mode == BB_CONV_DGRAD ? cin : cout;
    return dtype == BB_BF16 && (mode == BB_CONV_FWD || mode == BB_CONV_DGRAD) && n > 0 && h > 0 && w > 0 &&
           rows >= 128 && rows < (1ll << 31) && gathered >= 64 && gathered % 64 == 0 && produced % 8 == 0 &&
           produced >= 64;
}

extern "C" int bb_conv3x3(int dtype, int mode, int n, int h, int w, int cin, int cout, const void* src, const void* weight,
                          void* dst, float* strip_stats, void* stream) {
    BB_REQUIRE(src && weight && dst, "bb_conv3x3: null operand");
    BB_REQUIRE(!strip_stats || (mode == BB_CONV_FWD && ((uintptr_t)strip_stats % 16) == 0),
               "bb_conv3x3: strip_stats goes with BB_CONV_FWD only and must be 16-byte aligned");
    BB_REQUIRE(bb_conv3x3_supported(dtype, mode, n, h, w, cin, cout),
               "bb_conv3x3: unsupported problem (bf16, >= 128 pixels, gathered channels a multiple of 64, produced channels "
               "a multiple of 8 and >= 64): dtype %d mode %d n %d h %d w %d cin %d cout %d",
               dtype, mode, n, h, w, cin, cout);
    BB_REQUIRE(((uintptr_t)src % 16) == 0 && ((uintptr_t)weight % 16) == 0 && ((uintptr_t)dst % 16) == 0,
               "bb_conv3x3: operands must be 16-byte aligned");
    const bool dgrad = mode == BB_CONV_DGRAD;
    GemmArgs g = {};
    ConvArgs cv = {};
    g.M = n * h * w;
    g.N = dgrad ? cin : cout;
    g.K = 9 * (dgrad ? cout : cin);
    g.nb2 = 1;
    g.A = src;
    g.C = dst;
    g.lda = dgrad ? cout : cin;
    g.ldc = g.ldaux = g.N;
    g.alpha = 1.f;
    g.epilogue = BB_EPI_NONE;
    cv.h = h; cv.w = w; cv.c = dgrad ? cout : cin;
    hipStream_t st = (hipStream_t)stream;
    if (!dgrad) {
        // B = the weight as it lies: [cout, 9 * cin], k-contiguous
        g.B = weight;
        g.ldb = 9 * (int64_t)cin;
        if (strip_stats) {
            g.strip_stats = strip_stats;
            return launch_conv3x3<128, 64, 4, 2, false, 3, true>(g, cv, st);
        }
        // eight waves on a 128x64 tile (32x32 per wave): with one block per CU, two waves per SIMD hide each other's
        // LDS and barrier waits (four waves: 21.6 us, eight: 19.4 us at 6272 pixels, 256 channels)
        return launch_conv3x3<128, 64, 4, 2, false, 3>(g, cv, st);
    }
    // B[k = t * cout + o, n = i] = weight[o, 8 - t, i]: k-major with row stride 9 * cin, starting at tap 8; after
    // the cout / 64 k-tiles of a tap the rows go back to o = 0 and one tap down
    g.B = (const bf16*)weight + 8 * (int64_t)cin;
    g.ldb = 9 * (int64_t)cin;
    cv.b_every = cout / 64;
    cv.b_wrap = -(int64_t)cout * g.ldb - cin;
    return launch_conv3x3<64, 128, 2, 4, true, 3>(g, cv, st);
}

extern "C" int bb_conv3x3_dgrad_bn(int dtype, int n, int h, int w, int cin, int cout, const void* src, const void* weight, void* dst,
                                   const void* relu_out, const bb_bn_bwd_stats* bn, void* stream) {
    BB_REQUIRE(src && weight && dst, "bb_conv3x3_dgrad_bn: null operand");
    BB_REQUIRE(bb_conv3x3_supported(dtype, BB_CONV_DGRAD, n, h, w, cin, cout),
               "bb_conv3x3_dgrad_bn: unsupported problem (see bb_conv3x3): dtype %d n %d h %d w %d cin %d cout %d", dtype, n, h, w, cin, cout);
    BB_REQUIRE(((uintptr_t)src % 16) == 0 && ((uintptr_t)weight % 16) == 0 && ((uintptr_t)dst % 16) == 0 && ((uintptr_t)relu_out % 16) == 0,
               "bb_conv3x3_dgrad_bn: operands must be 16-byte aligned");
    int rc = check_bn_bwd_stats("bb_conv3x3_dgrad_bn", bn);
    if (rc) return rc;
    GemmArgs g = {};
    ConvArgs cv = {};
    g.M = n * h * w;
    g.N = cin;
    g.K = 9 * cout;
    g.nb2 = 1;
    g.A = src;
    g.C = dst;
    g.lda = cout;
    g.ldc = g.ldaux = g.N;
    g.alpha = 1.f;
    g.epilogue = relu_out ? BB_EPI_MUL_POS : BB_EPI_NONE;
    g.aux_in = relu_out;
    cv.h = h; cv.w = w; cv.c = cout;
    // the flipped filter read in place, as in bb_conv3x3
    g.B = (const bf16*)weight + 8 * (int64_t)cin;
    g.ldb = 9 * (int64_t)cin;
    cv.b_every = cout / 64;
    cv.b_wrap = -(int64_t)cout * g.ldb - cin;
    constexpr int BM = 64, BN = 128, STAGES = 3, smem = STAGES * (BM + BN) * 64 * 2;
    auto kern = conv3x3_bf16_igemm_bnbwd_kernel<BM, BN, 2, 4, STAGES>;
    BB_HIP_CHECK(bb_allow_dynamic_lds((const void*)kern, smem));
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    const BnBwdArgs b = {bn->x, bn->mean, bn->rstd, bn->strips};
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(2 * 4 * 64), smem, (hipStream_t)stream, g, cv, b);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

template <bool TA, bool TB, bool CONVB = false> static int launch_grouped(GroupedArgs& G, hipStream_t st) {
    constexpr int BM = 128, BN = 128, STAGES = 3;
    constexpr int smem = STAGES * (BM + BN) * 32 * 2;
    auto kern = gemm_bf16_dma_grouped_kernel<BM, BN, 2, 2, TA, TB, true, STAGES, CONVB>;
    BB_HIP_CHECK(bb_allow_dynamic_lds((const void*)kern, smem));
    int blocks = 0;
    for (int i = 0; i < G.count; ++i) {
        GemmArgs& g = G.p[i];
        g.tiles_m = (g.M + BM - 1) / BM;
        g.tiles_n = (g.N + BN - 1) / BN;
        G.first_block[i] = blocks;
        blocks += g.tiles_m * g.tiles_n;
    }
    G.first_block[G.count] = blocks;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), smem, st, G);
    BB_LAUNCH_CHECK();
    return BB_OK;
}

extern "C" int bb_gemm_grouped(const bb_gemm_desc* descs, int count, void* stream) {
    BB_REQUIRE(count >= 0 && (descs || count == 0), "bb_gemm_grouped: bad arguments");
    hipStream_t st = (hipStream_t)stream;
    // one launch when every problem is an unbatched bf16 problem of one layout that the DMA
    // kernel accepts; otherwise the problems run one after the other (same results)
    bool has_conv = false;
    for (int i = 0; i < count; ++i) has_conv = has_conv || descs[i].conv_c != 0;
    bool fuse = count >= (has_conv ? 1 : 2) && count <= GROUP_MAX;
    for (int i = 0; i < count && fuse; ++i) {
        const bb_gemm_desc& d = descs[i];
        // the grouped kernel is built without dropout decisions in its epilogue: such a problem runs by itself
        fuse = d.dtype == BB_BF16 && d.layout == descs[0].layout && d.nb1 <= 1 && d.nb2 <= 1 && d.M > 0 && d.N > 0 &&
               d.dropout_p == 0.f && pick_dma_tile(d.M, d.N, d.K, 1, d.layout) != D_NONE;
    }
    // fp32: unbatched problems of one layout that all take the small tile (each alone would leave CUs idle) share a launch
    bool fuse32 = !fuse && !has_conv && count >= 2 && count <= GROUP_MAX;
    for (int i = 0; i < count && fuse32; ++i) {
        const bb_gemm_desc& d = descs[i];
        fuse32 = d.dtype == BB_F32 && d.layout == descs[0].layout && d.nb1 <= 1 && d.nb2 <= 1 && d.M > 0 && d.N > 0 &&
                 d.dropout_p == 0.f && pick_f32_tile(d.M, d.N, 1) == 64;
    }
    if (fuse32) {
        GroupedArgs G;
        G.count = count;
        int blocks = 0;
        for (int i = 0; i < count; ++i) {
            int64_t batches;
            bool ta, tb;
            int rc = fill_args(&descs[i], G.p[i], batches, ta, tb);
            if (rc) return rc;
            // the bias gradient that rides on a weight gradient: its own kernel, as on the one-by-one route
            if (descs[i].colsum_out && (rc = colsum_standalone(&descs[i], stream)) != BB_OK) return rc;
            G.p[i].tiles_m = (G.p[i].M + 63) / 64;
            G.p[i].tiles_n = (G.p[i].N + 63) / 64;
            G.first_block[i] = blocks;
            blocks += G.p[i].tiles_m * G.p[i].tiles_n;
        }
        G.first_block[count] = blocks;
        const int layout = descs[0].layout;
        if (layout == BB_NT) hipLaunchKernelGGL((gemm_f32_grouped_kernel<false, false, 64>), dim3(blocks), dim3(256), 0, st, G);
        else if (layout == BB_NN) hipLaunchKernelGGL((gemm_f32_grouped_kernel<false, true, 64>), dim3(blocks), dim3(256), 0, st, G);
        else hipLaunchKernelGGL((gemm_f32_grouped_kernel<true, true, 64>), dim3(blocks), dim3(256), 0, st, G);
        BB_LAUNCH_CHECK();
        return BB_OK;
    }
    // a patch-matrix B exists only inside the grouped kernel: no one-by-one route for it
    BB_REQUIRE(fuse || !has_conv, "bb_gemm_grouped: a problem with a patch-matrix B must share a launch of bf16 BB_TN "
                                  "problems the DMA kernel takes (M, N >= 128, K %% 32 == 0)");
    if (!fuse) {
        for (int i = 0; i < count; ++i) {
            int rc = bb_gemm(&descs[i], stream);
            if (rc) return rc;
        }
        return BB_OK;
    }
    GroupedArgs G;
    G.count = count;
    for (int i = 0; i < count; ++i) {
        int64_t batches;
        bool ta, tb;
        int rc = fill_args(&descs[i], G.p[i], batches, ta, tb);
        if (rc) return rc;
        if (descs[i].colsum_out) G.p[i].colsum = descs[i].colsum_out;  // every grouped problem runs the DMA kernel
    }
    const int layout = descs[0].layout;
    if (layout == BB_NT) return launch_grouped<false, false>(G, st);
    if (layout == BB_NN) return launch_grouped<false, true>(G, st);
    if (has_conv) return launch_grouped<true, true, true>(G, st);
    return launch_grouped<true, true>(G, st);
}

// =========================================================================================
// Grouped GEMMs with few output tiles and a long contraction (the weight gradients of a ResNet
// bottleneck: 68 tiles of 128x128 over K = 6272 rows): the contraction is cut into `splits`
// chunks, each chunk of each problem becomes a problem of its own that writes an fp32 partial
// product into the caller's workspace, and a second kernel adds the partials to C in chunk order.
// =========================================================================================
constexpr int SPLITK_MAX = 8;

// every problem of the group in one launch: blockIdx.y = problem
struct SplitkReduceArgs {
    const float* ws[GROUP_MAX];
    float* C[GROUP_MAX];
    int64_t ldc[GROUP_MAX];
    int M[GROUP_MAX], N[GROUP_MAX], accumulate[GROUP_MAX];
    int splits;
};
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const SplitkReduceArgs a) {
    const int pi = blockIdx.y;
    const int M = a.M[pi], N = a.N[pi], splits = a.splits, accumulate = a.accumulate[pi];
    const float* __restrict__ ws = a.ws[pi];
    float* __restrict__ C = a.C[pi];
    const int64_t ldc = a.ldc[pi], part = (int64_t)M * N;
    const int64_t nvec = part / 4;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * 256) {
        const int64_t e = i * 4;
        const int m = (int)(e / N), n = (int)(e % N);
        float* c = C + (int64_t)m * ldc + n;
        f32x4 acc = accumulate ? *(const f32x4*)c : f32x4{0.f, 0.f, 0.f, 0.f};
        f32x4 v[SPLITK_MAX];
#pragma unroll
        for (int p = 0; p < SPLITK_MAX; ++p)
            if (p < splits) v[p] = *(const f32x4*)(ws + p * part + e);
#pragma unroll
        for (int p = 0; p < SPLITK_MAX; ++p)
            if (p < splits) acc += v[p];
        *(f32x4*)c = acc;
    }
}

// chunks of the contraction: 0 or 1 = run the group whole
static int pick_splits(const bb_gemm_desc* descs, int count) {
    if (count < 1 || count > GROUP_MAX) return 0;
    int64_t tiles = 0;
    int kmin = 1 << 30;
    for (int i = 0; i < count; ++i) {
        const bb_gemm_desc& d = descs[i];
        if (d.dtype != BB_BF16 || d.c_dtype != BB_F32 || d.layout != descs[0].layout || d.nb1 > 1 || d.nb2 > 1 || d.M <= 0 ||
            d.N <= 0 || d.colsum_out || d.bias || d.epilogue != BB_EPI_NONE || d.alpha != 1.0f || d.N % 4 != 0 || d.dropout_p != 0.f ||
            pick_dma_tile(d.M, d.N, d.K, 1, d.layout) == D_NONE)
            return 0;
        tiles += (int64_t)((d.M + 127) / 128) * ((d.N + 127) / 128);
        kmin = d.K < kmin ? d.K : kmin;
    }
    // Two blocks per CU on average: with one, a CU's four waves have nobody to hide their load and barrier waits
    // behind (the weight gradients of a ResNet block: 61.7 us at three chunks, 50.8 us at five).
    int splits = (int)(256 * 2 / tiles);
    if (splits > SPLITK_MAX) splits = SPLITK_MAX;
    if (splits > GROUP_MAX / count) splits = GROUP_MAX / count;
    while (splits > 1 && kmin / splits < 512) --splits;  // keep the pipelines of the chunks long
    return splits;
}

extern "C" int64_t bb_gemm_splitk_workspace(const bb_gemm_desc* descs, int count) {
    int64_t n = 0;
    for (int i = 0; descs && i < count; ++i) n += (int64_t)descs[i].M * descs[i].N;
    return n * SPLITK_MAX * (int64_t)sizeof(float);
}

extern "C" int bb_gemm_grouped_splitk(const bb_gemm_desc* descs, int count, void* workspace, int64_t workspace_bytes,
                                      void* stream) {
    BB_REQUIRE(count >= 0 && (descs || count == 0), "bb_gemm_grouped_splitk: bad arguments");
    const int splits = pick_splits(descs, count);
    if (splits <= 1) return bb_gemm_grouped(descs, count, stream);
    int64_t need = 0;
    for (int i = 0; i < count; ++i) need += (int64_t)descs[i].M * descs[i].N * splits * (int64_t)sizeof(float);
    BB_REQUIRE(workspace && workspace_bytes >= need && ((uintptr_t)workspace % 16) == 0,
               "bb_gemm_grouped_splitk: workspace of %lld bytes needed (16-byte aligned), got %lld", (long long)need,
               (long long)workspace_bytes);
    bb_gemm_desc sub[GROUP_MAX];
    float* ws = (float*)workspace;
    int ns = 0;
    for (int i = 0; i < count; ++i) {
        const bb_gemm_desc& d = descs[i];
        // chunk boundaries on multiples of 32 rows of the contraction
        const int kt = d.K / 32, per = kt / splits, extra = kt % splits;
        int k0 = 0;
        for (int p = 0; p < splits; ++p) {
            int kc = (per + (p < extra ? 1 : 0)) * 32;
            if (p == splits - 1) kc = d.K - k0;
            bb_gemm_desc& t = sub[ns++];
            t = d;
            t.K = kc;
            // A advances along its contraction index: rows for TN ([K, M]), columns otherwise ([M, K])
            t.A = (const char*)d.A + (d.layout == BB_TN ? (int64_t)k0 * d.lda : (int64_t)k0) * 2;
            // B: [N, K] for NT, [K, N] for NN and TN
            if (d.conv_c != 0) t.conv_row0 = d.conv_row0 + k0;   // the tensor stays put, the chunk starts k0 pixels in
            else t.B = (const char*)d.B + (d.layout == BB_NT ? (int64_t)k0 : (int64_t)k0 * d.ldb) * 2;
            t.C = ws + (int64_t)p * d.M * d.N;
            t.ldc = d.N;
            t.accumulate = 0;
            k0 += kc;
        }
        ws += (int64_t)splits * d.M * d.N;
    }
    int rc = bb_gemm_grouped(sub, ns, stream);
    if (rc) return rc;
    SplitkReduceArgs ra;
    ra.splits = splits;
    ws = (float*)workspace;
    int64_t most = 0;
    for (int i = 0; i < count; ++i) {
        const bb_gemm_desc& d = descs[i];
        const int64_t part = (int64_t)d.M * d.N;
        ra.ws[i] = ws; ra.C[i] = (float*)d.C; ra.ldc[i] = d.ldc;
        ra.M[i] = d.M; ra.N[i] = d.N; ra.accumulate[i] = d.accumulate;
        most = part / 4 > most ? part / 4 : most;
        ws += (int64_t)splits * part;
    }
    const unsigned bx = (unsigned)((most + 255) / 256 > 1024 ? 1024 : (most + 255) / 256);
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3(bx, (unsigned)count), dim3(256), 0, (hipStream_t)stream, ra);
    BB_LAUNCH_CHECK();
    return BB_OK;
}
