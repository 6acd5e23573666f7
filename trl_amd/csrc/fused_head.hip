// K5 / K6: lm_head fused with the log-prob / entropy reduction (forward) and its backward.
//
// All contractions run on the matrix cores (v_mfma_f32_32x32x16_{bf16,f16}, fp32 accumulate)
// through ONE "NT" tile loop: C[256 x 256] += A[256 x K] * B[256 x K]^T with both operands
// row-major and K contiguous, which is the layout the MFMA A/B fragments want (a lane holds 8
// consecutive k of one row), so fragments come straight out of LDS with 16-byte reads and nothing
// is ever transposed on the fly.  512 threads = 8 waves as 2 (M) x 4 (N); a wave owns 128 x 64 of
// the tile = 4 x 2 MFMA blocks = 128 accumulator registers per lane.  Tiles go from memory
// straight into a ring of LDS stages (global_load_lds_dwordx4) when K is a multiple of the k step,
// through registers otherwise.
//
// Forward (K5): the tile is computed TRANSPOSED -- M = vocabulary rows of W, N = tokens -- so that
// a lane of the accumulator layout holds 16 vocabulary entries of ONE token per block.  The online
// log-sum-exp state of a token therefore lives in the lane's own registers and the per-tile
// epilogue needs no cross-lane traffic; a workgroup keeps 256 tokens and walks over its share of
// the vocabulary tiles, the logits exist only as accumulators.
//
// Backward (K6), per vocabulary chunk: (1) dz = dL/dlogits as scaled fp16 [chunk, tokens] (vocabulary-major, each
// token's column in that token's own power-of-two scale) -- from a recompute of the chunk's logits (same tile loop),
// or, when the forward was asked to stash its softmax numerators, from one elementwise sweep over that stash;
// (2) dHidden += dz * W_chunk: the tile loop with dz as a K-MAJOR left operand (its k rows go to LDS as they lie in
// memory and the MFMA fragments come out through the LDS transpose loads, ds_read_b64_tr_b16) against W_chunk^T;
// (3) dW_chunk = dz^T * hidden as an NT product against hidden^T, whose columns carry the inverse of the tokens'
// scales; all on fp16 operands (bf16 inputs are converted while they are transposed).  The contraction of (2)/(3)
// is over a different axis than the recompute, and with H in the thousands the output tile of a fused kernel cannot
// stay in registers, so dz goes through a chunk-sized workspace (never the whole [N, V] matrix).
#include "common.hpp"

#include <type_traits>

namespace trlk {
namespace {

// Tile configuration (overridable with -D for experiments).
#ifndef TRLK_HEAD_BM
#define TRLK_HEAD_BM 256
#endif
#ifndef TRLK_HEAD_BN
#define TRLK_HEAD_BN 256
#endif
#ifndef TRLK_HEAD_BK
#define TRLK_HEAD_BK 64
#endif
#ifndef TRLK_HEAD_WGM
#define TRLK_HEAD_WGM 2
#endif
#ifndef TRLK_HEAD_WGN
#define TRLK_HEAD_WGN 4
#endif
constexpr int BM = TRLK_HEAD_BM, BN = TRLK_HEAD_BN, BK = TRLK_HEAD_BK;
constexpr int WGM = TRLK_HEAD_WGM, WGN = TRLK_HEAD_WGN;  // waves along M and N
constexpr int kHeadThreads = WGM * WGN * 64;
#ifndef TRLK_HEAD_WAVES_PER_EU
#define TRLK_HEAD_WAVES_PER_EU 2
#endif
#define TRLK_HEAD_KERNEL __global__ __launch_bounds__(kHeadThreads) __attribute__((amdgpu_waves_per_eu(TRLK_HEAD_WAVES_PER_EU, TRLK_HEAD_WAVES_PER_EU)))
constexpr int kLdsRow = BK + 8;  // elements per LDS row: 16 bytes of padding keep 16-byte reads conflict-free
constexpr int WM = BM / WGM, WN = BN / WGN;  // per-wave tile
constexpr int MB = WM / 32, NB = WN / 32;
constexpr int kCpr = BK / 8;                        // 16-byte chunks per tile row
constexpr int kRowStep = kHeadThreads / kCpr;       // rows staged per pass of the workgroup
constexpr int kLoadsA = BM / kRowStep, kLoadsB = BN / kRowStep;
constexpr int kTileABytes = BM * kLdsRow * 2, kTileBBytes = BN * kLdsRow * 2;
constexpr int kStageBytes = kTileABytes + kTileBBytes;
constexpr int kDirectLdsBytesDecl = 2 * (BM + BN) * 64 * 2;  // direct-to-LDS tile ring: 4 x 32-wide or 2 x 64-wide stages
constexpr int kDzLdsRow = BN * 2 + 16;     // bytes per vocabulary row of the dz tile staged in LDS by the backward
constexpr int cmax(int a, int b) { return a > b ? a : b; }
constexpr int kHeadLdsBytes = cmax(cmax(2 * kStageBytes, kDirectLdsBytesDecl), BM * kDzLdsRow);
static_assert(BM * kDzLdsRow <= kHeadLdsBytes, "dz staging tile");
static_assert(2 * WGM * BN * 4 * 4 <= kHeadLdsBytes && BN <= kHeadThreads, "merge scratch");
static_assert(BM % kRowStep == 0 && BN % kRowStep == 0 && WM % 32 == 0 && WN % 32 == 0 && BK % 16 == 0, "tile shape");

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int DT>
__device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    if constexpr (DT == TRLK_BF16)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                       0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                      0, 0);
}

// One operand of the NT product: `rows` x K, row-major with leading dimension ld (elements).  The left operand may
// instead be given "k-major" (AKM below): K x `rows`, row-major with leading dimension ld -- the transpose of what the
// product wants, read through the LDS transpose loads; its columns must be readable (and zero) up to the next
// multiple of the tile size.
struct Operand {
    const uint16_t* p;
    int64_t ld;
    int rows;
};
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

// k-step width of the direct-to-LDS loop per kernel.  All three use 64-wide steps (two 64 KiB stages, half as
// many barriers, whole 128-byte lines per row and step); the 32-wide, four-stage ring was only ahead for the
// short contraction over the hidden size while the forward's workgroups still ran out of step with each other.
#ifndef TRLK_HEAD_BK_FWD
#define TRLK_HEAD_BK_FWD 64
#endif
#ifndef TRLK_HEAD_BK_DZ
#define TRLK_HEAD_BK_DZ 64
#endif
#ifndef TRLK_HEAD_BK_GEMM
#define TRLK_HEAD_BK_GEMM 64
#endif

// Direct-to-LDS variant of the tile loop (K % BK == 0): `global_load_lds_dwordx4` moves 16 bytes per
// lane from memory straight into LDS, 1 KiB contiguous per wave instruction = 1024 / (2 BK) tile
// rows, with no register staging and no ds_write.  Rows are dense (no padding is possible inside a
// wave's 1 KiB), so bank conflicts are avoided by an XOR swizzle of the 16-byte chunk index: the
// chunk at physical position pc of row r holds logical chunk pc ^ swz(r), with
//   BK = 64 (128-byte rows): swz(r) = (r & 7) ^ ((r >> 3) & 1),   BK = 32 (64-byte rows): swz(r) = (r >> 2) & 3,
// which makes the 16 rows that one ds_read_b128 phase touches cover all 64 banks once.  The lane
// fetches that logical chunk from memory (a permutation inside one row, still coalesced) and the
// fragment reads apply the same XOR.
//
// The loop keeps kStages tiles in LDS (4 x 32 KiB for BK = 32, 2 x 64 KiB for BK = 64).  A stage is
// refilled as soon as the barrier that ends its last use has passed, kStages - 1 steps before it
// is needed again: the transfer of one stage through the CU's vector memory path (64 bytes per
// clock) takes longer than half a k step of MFMAs, so with only two stages every barrier waits
// for data in flight.
template <int BKT>
struct DirectCfg {
    static_assert(BKT == 32 || BKT == 64, "direct-to-LDS layouts exist for 32- and 64-wide k steps");
    static constexpr int kStages = BKT == 32 ? 4 : 2;
    static constexpr int kRowBytes = BKT * 2;                // dense LDS row
    static constexpr int kRowsPerBlk = 1024 / kRowBytes;     // rows one wave instruction fills
    static constexpr int kChunks = kRowBytes / 16;
    static constexpr int kDenseA = BM * kRowBytes, kDenseStage = (BM + BN) * kRowBytes;
    static constexpr int kLdsBytes = kStages * kDenseStage;
    static __device__ __forceinline__ int swizzle(int r) {
        return BKT == 64 ? ((r & 7) ^ ((r >> 3) & 1)) : ((r >> 2) & 3);
    }
};
static_assert(DirectCfg<32>::kLdsBytes <= kHeadLdsBytes && DirectCfg<64>::kLdsBytes <= kHeadLdsBytes, "LDS budget");

// Loader side of the direct-to-LDS loop: per-lane source offsets of the wave's tile blocks and the
// transfer of one stage.
// AKM: the left operand is k-major.  Its stage is then 64 k rows of 512 bytes (256 columns); one transfer fills two
// k rows; the 16-byte unit at physical position pu of k row r holds logical unit pu ^ ((r & 3) << 1), which spreads
// the four k rows that one group of 16 lanes reads with a transpose load over all banks.
template <int BKT, bool AKM = false>
struct DirectLoader {
    typedef DirectCfg<BKT> C;
    static_assert(!AKM || (BKT == 64 && BM == 256), "k-major left operands: 64-wide steps of 256 columns");
    static constexpr int kWaves = kHeadThreads / 64;
    static constexpr int kBlkA = BM / C::kRowsPerBlk / kWaves, kBlkB = BN / C::kRowsPerBlk / kWaves;  // per wave and stage
    static constexpr int kStageLoads = kBlkA + kBlkB;
    static_assert(BM % (C::kRowsPerBlk * kWaves) == 0 && BN % (C::kRowsPerBlk * kWaves) == 0, "blocks per wave");
    const char *abase, *bbase;
    char* smem;
    int wave;
    int64_t akstep;  // bytes between two k of the left operand
    uint32_t ao[kBlkA], bo[kBlkB];

    __device__ __forceinline__ DirectLoader(const Operand A, int m0, const Operand B, int n0, char* lds) : smem(lds) {
        const int lane = threadIdx.x & 63;
        wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: LDS targets stay scalar
        const int rr = lane / C::kChunks, pc = lane % C::kChunks;  // row inside a block, chunk position
        abase = reinterpret_cast<const char*>(AKM ? A.p + m0 : A.p + int64_t(m0) * A.ld);
        bbase = reinterpret_cast<const char*>(B.p + int64_t(n0) * B.ld);
        akstep = AKM ? A.ld * 2 : 2;
#pragma unroll
        for (int j = 0; j < kBlkA; ++j) {
            if constexpr (AKM) {
                const int krow = (wave + kWaves * j) * 2 + (lane >> 5);
                const int lu = (lane & 31) ^ ((krow & 3) << 1);  // the logical 16-byte unit this lane fetches
                ao[j] = uint32_t((int64_t(krow) * A.ld + lu * 8) * 2);
                continue;
            }
            const int row = (wave + kWaves * j) * C::kRowsPerBlk + rr;
            const int kc = pc ^ C::swizzle(row);  // the logical chunk this lane fetches
            const int r = m0 + row < A.rows ? row : A.rows - 1 - m0;
            ao[j] = uint32_t((int64_t(r) * A.ld + kc * 8) * 2);
        }
#pragma unroll
        for (int j = 0; j < kBlkB; ++j) {
            const int row = (wave + kWaves * j) * C::kRowsPerBlk + rr;
            const int kc = pc ^ C::swizzle(row);
            const int r = n0 + row < B.rows ? row : B.rows - 1 - n0;
            bo[j] = uint32_t((int64_t(r) * B.ld + kc * 8) * 2);
        }
    }
    // One 1 KiB transfer: 16 bytes per lane from `src` to LDS offset `lds` + 16 * lane.  Issued as
    // inline assembly on purpose: the compiler books a global_load_lds as an access of both memory
    // and LDS, after which every wait on a fragment read becomes lgkmcnt(0) (it stalls on the
    // reads just issued); the loop keeps its own vmcnt bookkeeping for these transfers anyway.
    // (m0 is a reserved register; naming it as clobbered is what tells the compiler not to keep a value there)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
    // The source is a uniform 64-bit base (scalar registers) plus the lane's 32-bit byte offset: one vector register
    // per transfer instead of an address pair, and the k step is added on the scalar side.
    static __device__ __forceinline__ void transfer(const char* base, uint32_t lane_off, uint32_t lds) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(lane_off),
                     "s"(reinterpret_cast<uint64_t>(base))
                     : "memory", "m0");
    }
#pragma clang diagnostic pop
    __device__ __forceinline__ uint32_t lds_base(int buf) const {
        return uint32_t(reinterpret_cast<uintptr_t>(smem)) + uint32_t(buf * C::kDenseStage);
    }
    // transfer j of a stage (A blocks first, then B blocks)
    __device__ __forceinline__ void issue_one(int buf, int k0, int j) const {
        if (j < kBlkA)
            transfer(abase + int64_t(k0) * akstep, ao[j], lds_base(buf) + (wave + kWaves * j) * 1024);
        else
            transfer(bbase + int64_t(k0) * 2, bo[j - kBlkA], lds_base(buf) + C::kDenseA + (wave + kWaves * (j - kBlkA)) * 1024);
    }
    __device__ __forceinline__ void issue(int buf, int k0) const {
#pragma unroll
        for (int j = 0; j < kStageLoads; ++j) issue_one(buf, k0, j);
    }
    // the first kStages tiles of a product; every stage must be free (all reads of the LDS done)
    __device__ __forceinline__ void prologue(int K) const {
        const int nk = K / BKT;
#pragma unroll
        for (int st = 0; st < C::kStages; ++st)
            if (st < nk) issue(st, st * BKT);
    }
};

// `prefetched`: the caller has already run DirectLoader::prologue for this tile (and nothing has
// touched the LDS since).
template <int DT, int BKT, bool AKM = false>
__device__ __forceinline__ void gemm_tile_nt_direct(const Operand A, int m0, const Operand B, int n0, int K,
                                                    f32x16 (&acc)[MB][NB], char* smem, bool prefetched) {
    typedef DirectCfg<BKT> C;
    constexpr int kStages = C::kStages, kRowBytes = C::kRowBytes;
    constexpr int kDenseA = C::kDenseA, kDenseStage = C::kDenseStage;
    const DirectLoader<BKT, AKM> loader(A, m0, B, n0, smem);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = loader.wave;
    const int wm = wave / WGN, wn = wave % WGN;

    // --- fragment side (tile rows of a wave start at multiples of 32, so the swizzle depends on the lane only)
    const int swz = C::swizzle(lane & 31);
    const int hl = lane >> 5;
    const int fa_row = (wm * WM + (lane & 31)) * kRowBytes, fb_row = (wn * WN + (lane & 31)) * kRowBytes;
    constexpr int KS = BKT / 16;
    int koff[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) koff[ks] = ((ks * 2 + hl) ^ swz) * 16;
    // k-major left operand: a fragment (32 rows x 16 k, 8 k per lane) is two transpose loads of 8 bytes.  The lanes
    // work in groups of 16: lane t of a group points at the 8 bytes that hold columns 4 (t % 4) .. + 3 of k row t / 4
    // (of the group's 4 k rows), and receives column t of those 4 k rows.  Groups 0, 1 take columns 0-15, 16-31 of the
    // block at k 0-3 (second load: 4-7), groups 2, 3 the same columns at k 8-11 (12-15).
    int fa_km[MB];
    if constexpr (AKM) {
        const int t = lane & 15, g = lane >> 4;
        const int f = (t >> 2) << 1;  // the unit swizzle of this lane's k row ((k row & 3) << 1)
        const int lu0 = (wm * WM + 16 * (g & 1)) / 8 + ((t & 3) >> 1);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
            fa_km[mb] = (8 * (g >> 1) + (t >> 2)) * 512 + ((lu0 + 4 * mb) ^ f) * 16 + (t & 1) * 8;
    }
    auto read_a = [&](const char* sa, int mb, int ks) -> u32x4 {
        if constexpr (AKM) {
            const uint32_t at = uint32_t(reinterpret_cast<uintptr_t>(sa)) + uint32_t(fa_km[mb] + ks * 16 * 512);
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_s16x4*>(at));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_s16x4*>(at + 4 * 512));
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            return __builtin_bit_cast(u32x4, both);
        } else {
            return *reinterpret_cast<const u32x4*>(sa + fa_row + mb * 32 * kRowBytes + koff[ks]);
        }
    };

#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mb][nb][r] = 0.f;

    // Software pipeline.  Fragment loads run one 16-wide k slice ahead of the MFMAs that consume them,
    // across the barrier too: the last slice of a stage is already in registers when the workgroup
    // synchronises, so its MFMAs cover the refill of the freed stage and the first fragment reads of
    // the next one.  The compiler's own scheduler sinks every ds_read next to its first use (one
    // exposed LDS latency per MFMA pair), so the issue order is pinned explicitly below.
    constexpr int kStageLoads = DirectLoader<BKT, AKM>::kStageLoads;
    auto load_frags = [&](int buf, int ks, u32x4(&fa)[MB], u32x4(&fb)[NB]) {
        const char* sa = smem + buf * kDenseStage;
        const char* sb = sa + kDenseA;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) fa[mb] = read_a(sa, mb, ks);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
            fb[nb] = *reinterpret_cast<const u32x4*>(sb + fb_row + nb * 32 * kRowBytes + koff[ks]);
    };
    u32x4 fa[2][MB], fb[2][NB];
    static_assert(KS % 2 == 0 && MB * NB > MB + NB && (kStages - 2) * kStageLoads < 64, "pipeline shape");
    constexpr std::true_type T{};
    constexpr std::false_type F{};
    const int nk = K / BKT;
    if (!prefetched) loader.prologue(K);
    if (nk >= kStages)
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kStages - 1) * kStageLoads) : "memory");
    else
        __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    load_frags(0, 0, fa[0], fb[0]);
    // Exact issue order, pinned instruction by instruction (sched_barrier(0) between the groups):
    // MFMA i of the slice, then at most one fragment read of the next slice and at most one tile
    // transfer.  Fragments are read in the order the mb-major MFMA sequence needs them (fa0, fb*,
    // fa1, ...), so every read has most of a slice between its issue and its first use.  The refill
    // of a stage is split: the first half of its transfers goes behind the barrier that frees it, the
    // second half into the first slice of the following step.
    constexpr int M = MB * NB, R = MB + NB;
    constexpr int kLoadsPost = (kStageLoads + 1) / 2, kLoadsPre = kStageLoads - kLoadsPost;
    auto slice = [&](u32x4(&ca)[MB], u32x4(&cb)[NB], auto read_tag, int rbuf, int rks, u32x4(&na)[MB], u32x4(&nb_)[NB],
                     auto nload_tag, int lbuf, int lk0, int lfirst) {
        constexpr bool READ = decltype(read_tag)::value;
        constexpr int NL = decltype(nload_tag)::value;
        const char* sa = smem + rbuf * kDenseStage;
        const char* sb = sa + kDenseA;
        int issued = 0;
#pragma unroll
        for (int i = 0; i < M; ++i) {
            const int mb = i / NB, nb = i % NB;
            acc[mb][nb] = mfma<DT>(ca[mb], cb[nb], acc[mb][nb]);
            if (READ && i < R) {
                // read order: fa[0], fb[0..NB-1], fa[1..MB-1]
                if (i == 0)
                    na[0] = read_a(sa, 0, rks);
                else if (i <= NB)
                    nb_[i - 1] = *reinterpret_cast<const u32x4*>(sb + fb_row + (i - 1) * 32 * kRowBytes + koff[rks]);
                else
                    na[i - NB] = read_a(sa, i - NB, rks);
            }
            if (NL > 0 && (i + 1) * NL / M > i * NL / M) {
                loader.issue_one(lbuf, lk0, lfirst + issued);
                ++issued;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    typedef std::integral_constant<int, kLoadsPost> post_t;
    typedef std::integral_constant<int, kLoadsPre> pre_t;
    typedef std::integral_constant<int, 0> zero_t;
    // POST / PRE: this step issues the first half of the refill of the stage it frees / the second
    // half of the refill the previous step started.  FULL, NEXT as above.
    auto xstep = [&](int kt, auto post_tag, auto pre_tag, auto full_tag, auto next_tag) {
        constexpr bool POST = decltype(post_tag)::value, PRE = decltype(pre_tag)::value;
        constexpr bool FULL = decltype(full_tag)::value, NEXT = decltype(next_tag)::value;
        const int cur = kt & (kStages - 1), prev = (kt - 1) & (kStages - 1);
#pragma unroll
        for (int ks = 0; ks + 1 < KS; ++ks) {
            if (PRE && ks == 0)
                slice(fa[ks & 1], fb[ks & 1], T, cur, ks + 1, fa[(ks + 1) & 1], fb[(ks + 1) & 1], pre_t{}, prev,
                      (kt - 1 + kStages) * BKT, kLoadsPost);
            else
                slice(fa[ks & 1], fb[ks & 1], T, cur, ks + 1, fa[(ks + 1) & 1], fb[(ks + 1) & 1], zero_t{}, 0, 0, 0);
        }
        // every fragment read of this stage has returned and the next stage has landed
        if constexpr (FULL)
            asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((kStages - 2) * kStageLoads) : "memory");
        else
            __builtin_amdgcn_s_waitcnt(0);
        // A bare s_barrier: __syncthreads() carries release/acquire fences, for which the compiler
        // drains every outstanding transfer (vmcnt(0)), younger stages included.  The waits above
        // are the ones this exchange needs; nothing may move across the barrier.
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" ::: "memory");
        constexpr int L = (KS - 1) & 1;
        const int nxt = (kt + 1) & (kStages - 1);
        if constexpr (NEXT && POST)
            slice(fa[L], fb[L], T, nxt, 0, fa[0], fb[0], post_t{}, cur, (kt + kStages) * BKT, 0);
        else if constexpr (NEXT)
            slice(fa[L], fb[L], T, nxt, 0, fa[0], fb[0], zero_t{}, 0, 0, 0);
        else
            slice(fa[L], fb[L], F, 0, 0, fa[0], fb[0], zero_t{}, 0, 0, 0);
    };
    static_assert(((KS - 1) & 1) == 1, "the last slice of a stage sits in fragment buffer 1, the next stage's first in 0");
    int kt = 0;
    if (nk > kStages) {
        xstep(kt++, T, F, T, T);
        for (; kt + kStages < nk; ++kt) xstep(kt, T, T, T, T);
        xstep(kt++, F, T, T, T);  // kt = nk - kStages: completes the last refill
    } else if (nk == kStages) {
        xstep(kt++, F, F, T, T);
    }
    for (; kt + 1 < nk; ++kt) xstep(kt, F, F, F, T);
    xstep(kt, F, F, F, F);
    // every LDS read of this tile completed before the last barrier: the caller may reuse the LDS right away
}

// acc[mb][nb] = sum_k A[m0 + .., k] * B[n0 + .., k].  Rows beyond the operand's end are clamped to
// its last row (callers ignore those outputs); k beyond K reads as zero (K % 8 == 0).
template <int DT>
__device__ __forceinline__ void gemm_tile_nt_staged(const Operand A, int m0, const Operand B, int n0, int K,
                                             f32x16 (&acc)[MB][NB], char* smem) {
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int kc = tid % kCpr, r0 = tid / kCpr;  // this thread stages rows r0 + kRowStep*j, 16-byte chunk kc

    // uniform tile base + 32-bit per-lane byte offsets (a tile spans < 4 GiB)
    const char* abase = reinterpret_cast<const char*>(A.p + int64_t(m0) * A.ld);
    const char* bbase = reinterpret_cast<const char*>(B.p + int64_t(n0) * B.ld);
    uint32_t ao[kLoadsA], bo[kLoadsB];
#pragma unroll
    for (int j = 0; j < kLoadsA; ++j) {
        int ra = r0 + kRowStep * j;
        ra = m0 + ra < A.rows ? ra : A.rows - 1 - m0;  // clamp to the operand's last row
        ao[j] = uint32_t((int64_t(ra) * A.ld + kc * 8) * 2);
    }
#pragma unroll
    for (int j = 0; j < kLoadsB; ++j) {
        int rb = r0 + kRowStep * j;
        rb = n0 + rb < B.rows ? rb : B.rows - 1 - n0;
        bo[j] = uint32_t((int64_t(rb) * B.ld + kc * 8) * 2);
    }
    const int st_off = (r0 * kLdsRow + kc * 8) * 2;        // + j * kRowStep rows
    const int fa_off = ((wm * WM + (lane & 31)) * kLdsRow + (lane >> 5) * 8) * 2;  // + mb*32 rows, + ks*16
    const int fb_off = ((wn * WN + (lane & 31)) * kLdsRow + (lane >> 5) * 8) * 2;

#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mb][nb][r] = 0.f;

    const u32x4 zero = {0u, 0u, 0u, 0u};
    // full k steps load unconditionally; only the last, partial step (K % BK != 0) masks its chunks
    auto load_stage = [&](u32x4(&ra)[kLoadsA], u32x4(&rb)[kLoadsB], int k0) {
        const char* ap = abase + int64_t(k0) * 2;
        const char* bp = bbase + int64_t(k0) * 2;
        if (k0 + BK <= K) {
#pragma unroll
            for (int j = 0; j < kLoadsA; ++j) ra[j] = *reinterpret_cast<const u32x4*>(ap + ao[j]);
#pragma unroll
            for (int j = 0; j < kLoadsB; ++j) rb[j] = *reinterpret_cast<const u32x4*>(bp + bo[j]);
        } else {
            const bool in = k0 + kc * 8 < K;
#pragma unroll
            for (int j = 0; j < kLoadsA; ++j) ra[j] = in ? *reinterpret_cast<const u32x4*>(ap + ao[j]) : zero;
#pragma unroll
            for (int j = 0; j < kLoadsB; ++j) rb[j] = in ? *reinterpret_cast<const u32x4*>(bp + bo[j]) : zero;
        }
    };
    auto store_stage = [&](const u32x4(&ra)[kLoadsA], const u32x4(&rb)[kLoadsB], int buf) {
        char* sa = smem + buf * kStageBytes;
        char* sb = sa + kTileABytes;
#pragma unroll
        for (int j = 0; j < kLoadsA; ++j) *reinterpret_cast<u32x4*>(sa + st_off + j * kRowStep * kLdsRow * 2) = ra[j];
#pragma unroll
        for (int j = 0; j < kLoadsB; ++j) *reinterpret_cast<u32x4*>(sb + st_off + j * kRowStep * kLdsRow * 2) = rb[j];
    };
    auto compute = [&](int buf) {
        const char* sa = smem + buf * kStageBytes;
        const char* sb = sa + kTileABytes;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            u32x4 fa[MB], fb[NB];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                fa[mb] = *reinterpret_cast<const u32x4*>(sa + fa_off + (mb * 32 * kLdsRow + ks * 16) * 2);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
                fb[nb] = *reinterpret_cast<const u32x4*>(sb + fb_off + (nb * 32 * kLdsRow + ks * 16) * 2);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = mfma<DT>(fa[mb], fb[nb], acc[mb][nb]);
        }
    };

    // Registers hold the tile of step kt+1 while step kt computes out of LDS; it is written to the
    // other LDS buffer at the end of the step (one barrier per step).
    const int nk = (K + BK - 1) / BK;
    u32x4 ra[kLoadsA], rb[kLoadsB];
    load_stage(ra, rb, 0);
    store_stage(ra, rb, 0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const bool more = kt + 1 < nk;
        if (more) load_stage(ra, rb, (kt + 1) * BK);
        compute(kt & 1);
        if (more) store_stage(ra, rb, (kt + 1) & 1);
        __syncthreads();
    }
}

template <int DT, int BKT, bool AKM = false>
__device__ __forceinline__ void gemm_tile_nt(const Operand A, int m0, const Operand B, int n0, int K,
                                             f32x16 (&acc)[MB][NB], char* smem, bool prefetched = false) {
    if constexpr (AKM) {  // (callers of this form pad K to whole steps)
        static_assert(BKT == 64, "k-major left operands need the direct-to-LDS loop with 64-wide steps");
        gemm_tile_nt_direct<DT, BKT, true>(A, m0, B, n0, K, acc, smem, prefetched);
    } else {
        if ((K & (BKT - 1)) == 0)
            gemm_tile_nt_direct<DT, BKT>(A, m0, B, n0, K, acc, smem, prefetched);
        else
            gemm_tile_nt_staged<DT>(A, m0, B, n0, K, acc, smem);
    }
}

// Row (M index) inside the workgroup tile of accumulator element r of block mb, for this lane.
__device__ __forceinline__ int acc_row(int wm, int mb, int r, int lane) {
    return wm * WM + mb * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
}
// Column (N index) inside the workgroup tile of block nb, for this lane.
__device__ __forceinline__ int acc_col(int wn, int nb, int lane) { return wn * WN + nb * 32 + (lane & 31); }

// Workgroup id -> (tile along axis `a`, tile along axis `b`) such that the workgroups that run
// together on one XCD (ids congruent mod 8, dispatched round-robin) form 4 x 8 patches: they share
// operand slabs through that XCD's L2.  An XCD owns the `a` tiles congruent to its number mod 8, in
// bands of 4; inside a band it walks b with the band's a tiles innermost.  The last band holds only
// as many a tiles per XCD as n_a needs, so that (almost) no workgroup of the grid is empty: the
// hardware deals workgroups to the CUs in order, and with empty ones interleaved at a fixed stride
// the real ones end up on a fraction of the CUs (measured: a third more time for 65 instead of 64
// a tiles with a grid padded to whole bands).  The n_a % 8 a tiles that are left when every XCD has
// the same number are not given to that many XCDs whole (one XCD in eight would then carry an a
// tile more than the others and the launch would wait for it): their n_b tiles each are dealt out
// in equal runs over all eight XCDs, a innermost.  The caller skips ta >= n_a or tb >= n_b.
__device__ __forceinline__ void xcd_patch(int w, int n_a, int n_b, int& ta, int& tb) {
    const int xcd = w & 7, q = w >> 3;
    const int groups = n_a >> 3;                   // a tiles every XCD owns whole
    const int bands = groups >> 2;                 // full bands of 4 of them
    const int full = bands * 4 * n_b;              // workgroups of this XCD in the full bands
    const int m = groups & 3;                      // whole a tiles per XCD in the last band
    if (q < full) {
        const int rem = q % (4 * n_b);
        tb = rem >> 2;
        ta = ((q / (4 * n_b)) * 4 + (rem & 3)) * 8 + xcd;
    } else if (q < full + m * n_b) {
        const int qq = q - full;
        tb = qq / m;
        ta = (bands * 4 + qq % m) * 8 + xcd;
    } else {
        const int r = (n_a & 7) ? (n_a & 7) : 1, left = (n_a & 7) * n_b;  // the a tiles that are left, and their tiles
        const int share = (left + 7) >> 3;
        const int t = xcd * share + (q - full - m * n_b);
        const bool real = q - full - m * n_b < share && t < left;
        ta = real ? groups * 8 + t % r : n_a;      // a innermost, as in the bands: neighbours share the b slab
        tb = real ? t / r : n_b;
    }
}
inline int xcd_patch_grid(int n_a, int n_b) {
    return 8 * ((n_a / 8) * n_b + ((n_a % 8) * n_b + 7) / 8);
}

// What a forward keeps for the backward when it is given a stash: for every logit its softmax numerator
//   e[v][n] = exp2(z[v][n] * log2(e) - ref) * 2^15   as fp16,   0 < e <= 2^15,
// where `ref` is the integer reference exponent that the lane which owned the logit held when it summed the tile
// (the running maximum of its part of the row, rounded up).  One reference covers the 64 rows of a 128-row block
// whose row quad (v / 4) has the same parity, for one token.  The backward's sweep turns a numerator into the
// probability with one multiplication: p = e * exp2(ref - 15 - log_z * log2(e)).  fp16 keeps 11 significant bits of
// every numerator down to 2^-29 of the running maximum and flushes below 2^-39 of it: the same accuracy d logits
// has after it is rounded to fp16 for the products, at half the bytes of the raw fp32 products.
//   quads  [vpad / 4][ld] x 8 bytes: the 4 rows of a quad for one token (rows are the vocabulary, vpad = V rounded up
//          to the tile; the accumulator layout gives a lane 4 consecutive rows of one token)
//   refs   [vpad / 128][2][ld] fp32: reference exponent of (128-row block, parity of the row quad, token)
//   zt     [ld] fp32: the target's logit z (a soft-capped head needs it for the chain factor of the one-hot term)
struct StashView {
    char* base;
    int64_t ld;    // tokens per row (>= N rounded up to the tile, or any with stash_cols)
    int64_t vpad;  // vocabulary rows the forward covered
    __host__ __device__ static int64_t rows8(int64_t vpad) { return vpad / 4 + vpad / 128 + 1; }  // rows of ld x 8 bytes
    __host__ __device__ uint2* quads() const { return reinterpret_cast<uint2*>(base); }
    __host__ __device__ float* refs() const { return reinterpret_cast<float*>(base + (vpad / 4) * ld * 8); }
    __host__ __device__ float* zt() const { return reinterpret_cast<float*>(base + (vpad / 4 + vpad / 128) * ld * 8); }
};

struct HeadArgs {
    const uint16_t* hidden;  // [N, H]
    const uint16_t* weight;  // [V, H]
    const int64_t* targets;  // [N]
    const float* bias;       // [V] added to hidden . weight[v] before scaling, or null
    int N, V, H;
    int64_t ldh, ldw;
    float logit_scale, inv_t, softcap;  // softcap <= 0: none
    // forward
    int v_splits, tiles_per_split;
    float* partial;  // [N, v_splits, 4]: (reference exponent, S, U, exact max of z)
    float* tgt;      // [N] logit of the target token (NaN until found)
    // backward (dz pass)
    const float* log_z;  // [N]
    const float* g;      // [N] upstream d loss / d logp
    int c0, c1;          // vocabulary rows of this chunk
    StashView stash;     // forward (written) and backward (read): the softmax numerators, or base == null
    const int32_t* stash_cols;  // backward: stash column of token n (tokens were compacted since the forward), or null
    uint16_t* dzT;       // [chunk rows padded, ldzt] (columns = tokens), fp16, column n scaled by pow2_scale(|g[n]| * zs)
    int64_t ldzt;
    const uint32_t* g_max;
    int sdz_token_blocks, sdz_tiles;  // stash sweep: token blocks per row group, tiles of the launch  // backward: bit pattern of max |g| over the tokens
};

// ---- scaled fp16 copies of the backward's operands -----------------------------------------------------------------
// The two backward products run on fp16 operands whatever the dtype of the problem: d logits rounded to bf16 would
// carry 8 significant bits into both gradients (relative error 3e-3), fp16 carries 11 (4e-4) at the same matrix-core
// rate.  fp16 has 5 exponent bits, so every operand is multiplied by a power of two that puts its largest magnitude
// into [2^13, 2^14) (exact, undone in the products' epilogue): d logits per token (|dz[:, n]| <= |g[n]| * logit_scale
// / T, so token n's column carries s_n = pow2_scale(|g[n]| * logit_scale / T) and a token whose upstream gradient is
// a million times smaller than the largest keeps its own relative accuracy in dHidden, whose row n the epilogue
// divides by s_n), W^T and hidden^T of a bf16 problem by their largest magnitude (bf16 -> fp16 is then exact down to
// 2^-31 of that maximum).  The dW product sums over the tokens, so it needs the columns of d logits in ONE scale: row
// n of hidden^T's source is multiplied by s_all / s_n on its way (s_all = the scale of the largest |g|, so the factor
// is a power of two <= 1), which leaves dz^T[v, n] * hidden^T[h, n] in the scale s_all * s_hidden for every n.  A token
// whose gradient is 2^-25 of the largest starts to lose bits of its hidden row there -- where its whole contribution
// to dW is below the rounding of the fp32 sum.
__device__ __forceinline__ float pow2_scale(float m) {
    if (!(m > 0.f) || !(m < INFINITY)) return 1.f;
    int e;
    (void)frexpf(m, &e);  // m = f * 2^e with f in [0.5, 1)
    int k = 14 - e;
    k = k > 100 ? 100 : (k < -100 ? -100 : k);
    return ldexpf(1.f, k);
}
__device__ __forceinline__ float slot_scale(const uint32_t* slot, float mult) {
    return slot != nullptr ? pow2_scale(__uint_as_float(*slot) * mult) : 1.f;
}

// tanh for soft-capping: sign(x) (1 - t) / (1 + t) with t = exp(-2 |x|) from the hardware's exp2 and reciprocal (a
// relative error of a few 1e-7), and the odd series x - x^3/3 + 2 x^5/15 below 0.05, where 1 - t cancels.  A third of
// the instructions of the library routine, in an epilogue that runs it once per logit.
__device__ __forceinline__ float head_tanh(float x) {
    const float ax = fabsf(x), x2 = x * x;
    const float t = fast_exp2(ax * (-2.f * kLog2e));
    const float big = (1.f - t) * __builtin_amdgcn_rcpf(1.f + t);
    const float small = ax * fmaf(x2, fmaf(x2, 2.f / 15.f, -1.f / 3.f), 1.f);
    return copysignf(ax < 0.05f ? small : big, x);
}

constexpr float kStashExp = 15.f;  // the numerators are summed and stashed times 2^15 (fp16's range above 1)

// GENERAL: soft-capping or a non-positive scale (z is computed per logit).  Otherwise z = (y + bias) * zs with one
// positive scale: the maximum is taken on the raw accumulators, the scale is folded into the exponent's multiplier and
// sum(e * z) is accumulated as zs * sum(e * y) -- the kernel of the usual head then carries no code of the other.
// STAGED: the hidden size is not a multiple of the direct-to-LDS loop's k step (a kernel of its own, so that the
// usual one does not carry the register-staged loop's code and loop-invariant registers through its tile loop).
template <int DT, bool STASH, bool GENERAL, bool STAGED>
TRLK_HEAD_KERNEL void fused_head_fwd_kernel(HeadArgs a) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int n_tb = (a.N + BN - 1) / BN;
    int tb, vs;
    xcd_patch(blockIdx.x, n_tb, a.v_splits, tb, vs);
    if (tb >= n_tb || vs >= a.v_splits) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int n0 = tb * BN;
    const int n_vt = (a.V + BM - 1) / BM;
    const int vt0 = vs * a.tiles_per_split;
    const int vt1 = vt0 + a.tiles_per_split < n_vt ? vt0 + a.tiles_per_split : n_vt;

    // per-lane online state of the NB tokens this lane owns (base-2, integer reference exponent)
    float ref[NB], rr[NB], S[NB], U[NB], zmax[NB];
    int64_t tg[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        ref[nb] = -INFINITY;
        zmax[nb] = -INFINITY;
        rr[nb] = 0.f;
        S[nb] = 0.f;
        U[nb] = 0.f;
        const int tok = n0 + acc_col(wn, nb, lane);
        tg[nb] = tok < a.N ? a.targets[tok] : -1;
    }
    const Operand W{a.weight, a.ldw, a.V}, Hd{a.hidden, a.ldh, a.N};

    if constexpr (!STAGED)
        if (vt0 < vt1) DirectLoader<TRLK_HEAD_BK_FWD>(W, vt0 * BM, Hd, n0, smem).prologue(a.H);
    for (int vt = vt0; vt < vt1; ++vt) {
        const int m0 = vt * BM;
        f32x16 acc[MB][NB];
        if constexpr (STAGED) {
            gemm_tile_nt_staged<DT>(W, m0, Hd, n0, a.H, acc, smem);
        } else {
            gemm_tile_nt_direct<DT, TRLK_HEAD_BK_FWD>(W, m0, Hd, n0, a.H, acc, smem, true);
            // the next tile's first stages travel while this tile's logits are reduced (registers only)
            if (vt + 1 < vt1) DirectLoader<TRLK_HEAD_BK_FWD>(W, m0 + BM, Hd, n0, smem).prologue(a.H);
        }
        // Stash: for one accumulator quad (4 consecutive vocabulary rows of one token per lane) the 32 lanes of a
        // half-wave hold 32 consecutive tokens = 256 contiguous bytes per store.  The buffer is padded to whole tiles.
        // Addresses are a uniform pointer that walks down the quads (scalar registers, one addition per store) plus
        // the lane's byte offset (one vector register; the entry point bounds ld so that it fits 32 bits).
        char* stash_blk = nullptr;
        float* ref_blk = nullptr;
        uint32_t stash_lane = 0, ref_lane = 0;
        if constexpr (STASH) {
            const int uw = __builtin_amdgcn_readfirstlane(wave);
            const int uwm = uw / WGN, ucol = n0 + (uw % WGN) * WN;
            stash_blk = reinterpret_cast<char*>(a.stash.quads() + int64_t(m0 / 4 + uwm * (WM / 4)) * a.stash.ld + ucol);
            ref_blk = a.stash.refs() + int64_t(m0 / 128 + uwm) * 2 * a.stash.ld + ucol;
            ref_lane = uint32_t(lane >> 5) * uint32_t(a.stash.ld) + uint32_t(lane & 31);
            stash_lane = ref_lane * 8u;
        }
        const bool partial_tile = m0 + BM > a.V;
        const float zs = a.logit_scale * a.inv_t, zs2 = zs * kLog2e;
        constexpr bool plain = !GENERAL;
        // Before the reduction, only where needed (a bias, the general form of z, or the vocabulary's last tile, whose
        // rows beyond the vocabulary count as -inf): the accumulators become y + bias (usual head) or z itself
        // (general form).  A lane's 16 accumulators of a block are 4 quads of consecutive vocabulary rows, so the bias
        // comes as one 16-byte load per quad, all of a block row's loads issued before the first is used.
        if (GENERAL || a.bias != nullptr || partial_tile) {
            const float inv_cap = a.softcap > 0.f ? 1.f / a.softcap : 0.f;
            typedef float f32x4_dword_aligned __attribute__((ext_vector_type(4), aligned(4)));
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                f32x4 bq[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int v0 = m0 + acc_row(wm, mb, q * 4, lane);
                    bq[q] = f32x4{0.f, 0.f, 0.f, 0.f};
                    if (a.bias != nullptr) {
                        if (v0 + 3 < a.V) {
                            bq[q] = *reinterpret_cast<const f32x4_dword_aligned*>(a.bias + v0);
                        } else {
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                if (v0 + i < a.V) bq[q][i] = a.bias[v0 + i];
                        }
                    }
                }
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int v0 = m0 + acc_row(wm, mb, q * 4, lane);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const bool beyond = partial_tile && v0 + i >= a.V;
#pragma unroll
                        for (int nb = 0; nb < NB; ++nb) {
                            float y = acc[mb][nb][q * 4 + i] + bq[q][i];
                            if constexpr (GENERAL) {
                                y *= a.logit_scale;
                                if (a.softcap > 0.f) y = head_tanh(y * inv_cap) * a.softcap;
                                y *= a.inv_t;
                            }
                            acc[mb][nb][q * 4 + i] = beyond ? -INFINITY : y;
                        }
                    }
                }
            }
        }
        // (With a stash the numerators are stored as they are produced.  Packed into registers and stored in one run
        // at the end of the epilogue they cost more: 28.6 against 27.8 ms for the benchmark's forward.)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            float bm = -INFINITY;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) bm = fmaxf(bm, acc[mb][nb][r]);
            if constexpr (plain) bm *= zs;
            // target logit: rarely inside this wave's 128 vocabulary rows.  It is selected into one register
            // and stored once: a conditional store per accumulator held the wave for about 20 us, and a
            // workgroup that falls behind the others no longer finds the tiles they share in the L2.
            const int64_t rel = tg[nb] - (m0 + wm * WM);
            if (rel >= 0 && rel < WM) {
                const int want = int(rel) - (lane >> 5) * 4;  // acc_row() without this lane's half-wave offset
                float tv = 0.f;
                bool mine = false;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const bool m = (mb * 32 + (r >> 2) * 8 + (r & 3)) == want;
                        tv = m ? acc[mb][nb][r] : tv;
                        mine |= m;
                    }
                if (mine) a.tgt[n0 + acc_col(wn, nb, lane)] = plain ? tv * zs : tv;
            }
            zmax[nb] = fmaxf(zmax[nb], bm);
            const float need = ceilf(bm * kLog2e);
            if (need > ref[nb]) {
                const float sc = fast_exp2(ref[nb] - need);
                S[nb] *= sc;
                U[nb] *= sc;
                ref[nb] = need;
                rr[nb] = need;
            }
            // numerators times 2^15 (exact; S and U carry the factor until they are written out), with or without a
            // stash: the outputs must not depend on stashing
            int64_t stash_off = nb * 32 * 8;  // byte offset of this token block's column of quads (uniform)
            if constexpr (STASH) ref_blk[nb * 32 + ref_lane] = rr[nb];
            const float rsub = rr[nb] - kStashExp;
            float s = 0.f, u = 0.f;
            auto sum_tile = [&](auto guard_tag) {
                constexpr bool kGuard = decltype(guard_tag)::value;  // -inf among the logits (0 * -inf in sum(e * y))
                const float mul = plain ? zs2 : kLog2e;  // general path: the accumulators hold z itself by now
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        float e[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const float y = acc[mb][nb][q * 4 + i];
                            e[i] = fast_exp2(fmaf(y, mul, -rsub));
                            s += e[i];
                            u = (kGuard && y == -INFINITY) ? u : fmaf(e[i], y, u);
                        }
                        if constexpr (STASH) {
                            uint2 w;
                            w.x = Elem<TRLK_F16>::pack2(e[0], e[1]);
                            w.y = Elem<TRLK_F16>::pack2(e[2], e[3]);
                            *reinterpret_cast<uint2*>(stash_blk + stash_off + stash_lane) = w;
                            stash_off += a.stash.ld * 16;  // two quads down: the other parity is the other half-wave's
                            // (one running offset, not 16 precomputed ones; an offset, because a pointer that
                            // passed through here would no longer be known to point to global memory)
                            asm volatile("" : "+s"(stash_off));
                        }
                    }
            };
            if (GENERAL || partial_tile)
                sum_tile(std::true_type{});
            else
                sum_tile(std::false_type{});
            if constexpr (plain) u *= zs;
            S[nb] += s;
            U[nb] += u;
        }
    }

    // merge the partial states of every token (2 lane halves x WGM M-waves) through LDS
    constexpr int kParts = 2 * WGM;
    float* sm = reinterpret_cast<float*>(smem);  // [kParts][BN tokens][4]
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int col = acc_col(wn, nb, lane);
        const int part = wm * 2 + (lane >> 5);
        float* dst = sm + (part * BN + col) * 4;
        dst[0] = ref[nb];
        dst[1] = S[nb] * 0x1p-15f;
        dst[2] = U[nb] * 0x1p-15f;
        dst[3] = zmax[nb];
    }
    __syncthreads();
    if (tid < BN && n0 + tid < a.N) {
        float R = -INFINITY;
        float zm = -INFINITY;
        for (int p = 0; p < kParts; ++p) {
            R = fmaxf(R, sm[(p * BN + tid) * 4]);
            zm = fmaxf(zm, sm[(p * BN + tid) * 4 + 3]);
        }
        float s = 0.f, u = 0.f;
        for (int p = 0; p < kParts; ++p) {
            const float* src = sm + (p * BN + tid) * 4;
            const float sc = (src[0] == -INFINITY) ? 0.f : fast_exp2(src[0] - R);
            s += src[1] * sc;
            u += src[2] * sc;
        }
        float* out = a.partial + (int64_t(n0 + tid) * a.v_splits + vs) * 4;
        out[0] = R;
        out[1] = s;
        out[2] = u;
        out[3] = zm;
    }
}

__global__ void head_fill_kernel(float* p, int64_t n, float v) {
    const int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// merges the vocabulary splits of every token: logp, entropy, log_z
__global__ void head_merge_kernel(const float* partial, const float* tgt, const int64_t* targets, int N, int V,
                                  int v_splits, float* logp, float* entropy, float* log_z, float* target_is_max,
                                  int32_t* error_flag, float* stash_zt) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= N) return;
    const float* p = partial + int64_t(n) * v_splits * 4;
    float R = -INFINITY;
    for (int s = 0; s < v_splits; ++s) R = fmaxf(R, p[s * 4]);
    float S = 0.f, U = 0.f, zm = -INFINITY;
    for (int s = 0; s < v_splits; ++s) {
        zm = fmaxf(zm, p[s * 4 + 3]);
        const float sc = (p[s * 4] == -INFINITY) ? 0.f : fast_exp2(p[s * 4] - R);
        S += p[s * 4 + 1] * sc;
        U += p[s * 4 + 2] * sc;
    }
    constexpr float kLn2Hi = 0.693145751953125f, kLn2Lo = 1.42860677e-06f;
    const float lz = fmaf(R, kLn2Hi, fmaf(R, kLn2Lo, logf(S)));
    const int64_t t = targets[n];
    float lp;
    if (t < 0 || t >= V) {
        lp = NAN;
        if (error_flag) atomicOr(error_flag, TRLK_FLAG_INDEX_OUT_OF_RANGE);
    } else {
        lp = tgt[n] - lz;
    }
    logp[n] = lp;
    if (stash_zt) stash_zt[n] = tgt[n];
    entropy[n] = lz - U / S;
    log_z[n] = lz;
    // 1 if the target holds the row maximum, i.e. argmax(logits) == target up to ties
    if (target_is_max) target_is_max[n] = (t >= 0 && t < V && tgt[n] >= zm) ? 1.f : 0.f;
}

// dz pass of the backward: one 256 (vocabulary) x 256 (tokens) tile per workgroup.
template <int DT>
TRLK_HEAD_KERNEL void fused_head_dz_kernel(HeadArgs a) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int n_tb = (a.N + BN - 1) / BN;
    const int n_vt = (a.c1 - a.c0 + BM - 1) / BM;
    int tb, vt;
    xcd_patch(blockIdx.x, n_tb, n_vt, tb, vt);
    if (tb >= n_tb || vt >= n_vt) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int n0 = tb * BN, m0 = a.c0 + vt * BM;
    const Operand W{a.weight, a.ldw, a.V}, Hd{a.hidden, a.ldh, a.N};
    f32x16 acc[MB][NB];
    gemm_tile_nt<DT, TRLK_HEAD_BK_DZ>(W, m0, Hd, n0, a.H, acc, smem);

    // Common case (no soft-capping, tile inside the chunk): dz = -(g * chain) * exp2(y * zs2 - lzc)
    // with one scale folded into the exponent; the target's one-hot term is patched afterwards.
    const float zs = a.logit_scale * a.inv_t, zs2 = zs * kLog2e;
    const bool plain = a.softcap <= 0.f && m0 + BM <= a.c1 && a.bias == nullptr;
    typedef Elem<TRLK_F16> EO;  // storage of dz
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int tok = n0 + acc_col(wn, nb, lane);
        const bool tok_ok = tok < a.N;
        const float g = tok_ok ? a.g[tok] * pow2_scale(fabsf(a.g[tok]) * zs) : 0.f;  // g carries the token's scale
        const float lzc = tok_ok ? a.log_z[tok] * kLog2e : INFINITY;  // rows beyond N: exp2(-inf) = 0
        const int64_t tg = tok_ok ? a.targets[tok] : -1;
        const int64_t rel = tg - (m0 + wm * WM);  // target row relative to this wave's rows
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            float d[16];
            if (plain) {
                const float ngc = -g * zs;
#pragma unroll
                for (int r = 0; r < 16; ++r) d[r] = ngc * fast_exp2(fmaf(acc[mb][nb][r], zs2, -lzc));
                if (rel >= mb * 32 && rel < mb * 32 + 32) {
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        if (acc_row(0, mb, r, lane) == int(rel)) d[r] -= ngc;
                }
            } else {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int v = m0 + acc_row(wm, mb, r, lane);
                    float y = acc[mb][nb][r];
                    if (a.bias != nullptr && v < a.c1) y += a.bias[v];
                    y *= a.logit_scale;
                    float chain = a.inv_t * a.logit_scale;
                    if (a.softcap > 0.f) {
                        const float th = head_tanh(y / a.softcap);
                        y = th * a.softcap;
                        chain *= 1.f - th * th;
                    }
                    const float z = y * a.inv_t;
                    const float p = fast_exp2(fmaf(z, kLog2e, -lzc));
                    float dzv = -g * p;
                    if (v == tg) dzv += g;
                    d[r] = (v < a.c1 && tok_ok) ? dzv * chain : 0.f;
                }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mb][nb][r] = d[r];
        }
    }
    // dz^T [chunk row][token]: the lanes of a block hold consecutive tokens of one vocabulary row.
    // Neighbouring lanes swap one value each, so that the even lane owns two tokens of row r and
    // the odd lane two tokens of row r + 1; the 4-byte pieces are staged as a [vocabulary][token]
    // tile in LDS and leave as 512-byte runs.
    constexpr int kChunksPerRow = BN / 8;  // 16-byte pieces per row of the staged tile
    const int odd = lane & 1;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int tcol = (acc_col(wn, nb, lane) & ~1) * 2;  // byte offset of the token pair inside a staged row
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                const float mine0 = acc[mb][nb][r], mine1 = acc[mb][nb][r + 1];
                const float give = odd ? mine0 : mine1;
                const float got = __builtin_bit_cast(
                    float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, give), 0xB1 /* quad_perm 1,0,3,2 */, 0xf, 0xf, true));
                const uint32_t w = odd ? EO::pack2(got, mine1) : EO::pack2(mine0, got);
                const int vrow = acc_row(wm, mb, r, lane) + odd;
                *reinterpret_cast<uint32_t*>(smem + vrow * kDzLdsRow + tcol) = w;
            }
    }
    __syncthreads();
#pragma unroll 4
    for (int c = tid; c < BM * kChunksPerRow; c += kHeadThreads) {
        const int vrow = c / kChunksPerRow, tc = c % kChunksPerRow;  // chunk-local row (padding rows are written as 0)
        *reinterpret_cast<u32x4*>(a.dzT + int64_t(vt * BM + vrow) * a.ldzt + n0 + tc * 8) =
            *reinterpret_cast<const u32x4*>(smem + vrow * kDzLdsRow + tc * 16);
    }
}

// dz pass of the backward from the forward's stashed softmax numerators instead of a recompute: an
// elementwise sweep (memory bound: 2 bytes read, 2 bytes written per logit, one multiplication each).
// One workgroup = 128 vocabulary rows x 256 tokens.  A lane owns two pairs of tokens, a wave 32 rows = 8 row quads
// whose 16 loads (16 bytes each: 2 tokens x 4 rows) are all issued before the first result is used.
// dz^T (vocabulary-major, like the stash) is written in place, each token's column in that token's own scale.
// Rows beyond the chunk and tokens beyond N are written as zeros.
constexpr int kSdzRows = 128, kSdzTokens = 256, kSdzQuads = kSdzRows / 4 / 4;  // quads per wave
// COLS: the tokens were compacted since the forward, a.stash_cols maps them to their stash columns.
// CAPPED: soft-capped head (the chain factor needs the logit: a logarithm per numerator); a kernel of its own, so that
// the usual sweep is straight-line code.
template <bool COLS, bool CAPPED>
__global__ __launch_bounds__(256) void head_dz_from_stash_kernel(HeadArgs a) {
    typedef Elem<TRLK_F16> E;  // the numerators and dz are fp16
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // consecutive tiles take consecutive token blocks of one row group: the stash rows they read and the
    // dz^T rows they write are then neighbours in memory.  Consecutive workgroups go to the eight XCDs in turn:
    // each XCD walks one contiguous eighth of the tiles.
    const int per_xcd = int(gridDim.x) >> 3;  // (the grid is a multiple of 8)
    const int tile = int(blockIdx.x & 7) * per_xcd + int(blockIdx.x >> 3);
    if (tile >= a.sdz_tiles) return;
    const int n0 = (tile % a.sdz_token_blocks) * kSdzTokens, r0 = (tile / a.sdz_token_blocks) * kSdzRows;  // r0: chunk-local row
    const int rows = a.c1 - a.c0;
    const float zs = a.logit_scale * a.inv_t;
    const int64_t ld = a.stash.ld;
    // A lane owns two pairs of neighbouring tokens, 128 apart: every load instruction of the wave then reads 1 KiB of
    // one stash row without gaps (16 bytes = 2 tokens x 4 rows per lane), every store 256 contiguous bytes of a dz row.
    const int tl[4] = {lane * 2, lane * 2 + 1, 128 + lane * 2, 128 + lane * 2 + 1};
    float ngc[4], lzc[4];  // -g * zs in the token's own scale; log_z in base 2
    int tg[4], col[4];     // chunk-local target row (or -1); stash column
    bool live[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int tok = n0 + tl[j];
        const bool ok = tok < a.N;
        col[j] = ok ? (COLS ? a.stash_cols[tok] : tok) : -1;
        const float g = ok ? a.g[tok] : 0.f;
        live[j] = g != 0.f;
        ngc[j] = -g * pow2_scale(fabsf(g) * zs) * zs;
        lzc[j] = ok ? a.log_z[tok] * kLog2e : INFINITY;
        const int64_t t = ok ? a.targets[tok] - a.c0 : -1;
        tg[j] = (t >= 0 && t < rows) ? int(t) : -1;
    }
    // (tokens beyond N of the last block are inside the padded row)
    const bool pair0 = !COLS || (col[0] >= 0 && col[1] == col[0] + 1), pair1 = !COLS || (col[2] >= 0 && col[3] == col[2] + 1);
    const int c0 = COLS ? col[0] : n0 + tl[0], c2 = COLS ? col[2] : n0 + tl[2];
    // the numerators of the wave's 8 quads
    const int row_w = r0 + wave * (kSdzRows / 4);                         // chunk-local first row of the wave
    const uint2* qrow = a.stash.quads() + int64_t((a.c0 + row_w) / 4) * ld;  // (chunks and tiles start on whole 128-row blocks)
    uint2 eb[kSdzQuads][4];
#pragma unroll
    for (int qi = 0; qi < kSdzQuads; ++qi) {
        const uint2* src = qrow + int64_t(qi) * ld;
        typedef uint32_t u32x4_8 __attribute__((ext_vector_type(4), aligned(8)));
        if (pair0) {
            const u32x4_8 lo = __builtin_nontemporal_load(reinterpret_cast<const u32x4_8*>(src + c0));
            eb[qi][0] = make_uint2(lo.x, lo.y);
            eb[qi][1] = make_uint2(lo.z, lo.w);
        } else {
#pragma unroll
            for (int j = 0; j < 2; ++j) eb[qi][j] = col[j] >= 0 ? src[col[j]] : make_uint2(0u, 0u);
        }
        if (pair1) {
            const u32x4_8 hi = __builtin_nontemporal_load(reinterpret_cast<const u32x4_8*>(src + c2));
            eb[qi][2] = make_uint2(hi.x, hi.y);
            eb[qi][3] = make_uint2(hi.z, hi.w);
        } else {
#pragma unroll
            for (int j = 2; j < 4; ++j) eb[qi][j] = col[j] >= 0 ? src[col[j]] : make_uint2(0u, 0u);
        }
    }
    // reference exponents of the two quad parities -> the factor that turns a numerator into -g * zs * p
    const float* refs = a.stash.refs() + int64_t((a.c0 + row_w) / 128) * 2 * ld;
    float rf[2][4], pf[2][4];  // p = e * pf
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int cj = COLS ? col[j] : n0 + tl[j];
            rf[h][j] = (COLS && cj < 0) ? 0.f : refs[int64_t(h) * ld + cj];
            pf[h][j] = fast_exp2(rf[h][j] - kStashExp - lzc[j]);
        }
    constexpr bool capped = CAPPED;
    float zt[4] = {0.f, 0.f, 0.f, 0.f};
    if constexpr (capped) {
#pragma unroll
        for (int j = 0; j < 4; ++j) zt[j] = col[j] >= 0 ? a.stash.zt()[col[j]] : 0.f;
    }
    const float th_mul = capped ? 1.f / (a.inv_t * a.softcap) : 0.f;  // tanh(.) of a soft-capped logit = z * T / cap
#pragma unroll
    for (int qi = 0; qi < kSdzQuads; ++qi) {
        const int h = qi & 1;  // (the wave's first quad is even)
        float e[4][4];         // [token][row of the quad]
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            E::unpack2(eb[qi][j].x, &e[j][0]);
            E::unpack2(eb[qi][j].y, &e[j][2]);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = row_w + qi * 4 + i;
            float d[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float p = e[j][i] * pf[h][j];
                float dv;
                if constexpr (!capped) {
                    dv = ngc[j] * p;
                    if (tg[j] == row) dv -= ngc[j];
                } else {
                    // z from the numerator (a flushed one has p = 0 and, unless it is the target, no gradient)
                    const bool is_t = tg[j] == row;
                    const float z = is_t ? zt[j] : (__log2f(e[j][i]) - kStashExp + rf[h][j]) * kLn2;
                    const float th = z * th_mul;
                    dv = ngc[j] * (is_t ? p - 1.f : p) * (1.f - th * th);
                    if (!is_t && e[j][i] == 0.f) dv = 0.f;
                }
                d[j] = (row < rows && live[j]) ? dv : 0.f;
            }
            // (non-temporal: 2 GB per chunk that no cache holds until the products read it)
            uint32_t* out = reinterpret_cast<uint32_t*>(a.dzT + int64_t(row) * a.ldzt + n0);
            __builtin_nontemporal_store(E::pack2(d[0], d[1]), out + lane);
            __builtin_nontemporal_store(E::pack2(d[2], d[3]), out + 64 + lane);
        }
    }
}

// Plain NT product with an output epilogue: C[M, N] (+)= A[M, K] * B[N, K]^T.
//   MODE 0: store to `out_lp` in the storage dtype.
//   MODE 1: fp32 accumulate into `out_f32` (first = overwrite).
//   MODE 2: like 1 but the sum is rounded into `out_lp` instead of being written back (last chunk).
//   The accumulators are multiplied by 1 / (scale of A * scale of B) first: the scales are powers of two derived from
//   the maxima in `max_a` (times `mult_a`) and `max_b` (null = 1), and, when `g_rows` is given, row m of A carries its
//   own scale pow2_scale(|g_rows[m]| * mult_a) instead of the common one.
struct GemmArgs {
    Operand A, B;
    int M, N, K;
    float* out_f32;
    int64_t ld_f32;
    uint16_t* out_lp;
    int64_t ld_lp;
    int first;
    const uint32_t* max_a;
    const uint32_t* max_b;
    const float* g_rows;
    float mult_a;
};

// DT: dtype of the operands (the matrix-core instruction), ODT: storage dtype of `out_lp`.
// AKM: A is given k-major ([K, M], leading dimension A.ld).
template <int DT, int MODE, int ODT, bool AKM = false>
__device__ __forceinline__ void gemm_nt_body(const GemmArgs& a, int block, char* smem) {
    typedef Elem<ODT> E;
    const int n_mt = (a.M + BM - 1) / BM, n_nt = (a.N + BN - 1) / BN;
    int tm, tn;
    xcd_patch(block, n_mt, n_nt, tm, tn);
    if (tm >= n_mt || tn >= n_nt) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int m0 = tm * BM, n0 = tn * BN;
    f32x16 acc[MB][NB];
    gemm_tile_nt<DT, TRLK_HEAD_BK_GEMM, AKM>(a.A, m0, a.B, n0, a.K, acc, smem);
    const float inv_b = 1.f / slot_scale(a.max_b, 1.f);
    const float inv_common = inv_b / slot_scale(a.max_a, a.mult_a);
    // A tile inside the output (nearly every tile): no per-element predicates, addresses as a uniform base plus one
    // 32-bit lane offset, the 16 running sums of a block loaded before the first is used and its 16 results stored in
    // one run.  (Written per element with a bounds test each, the compiler lost count of the loads in flight and
    // waited for EVERYTHING outstanding before each accumulate, i.e. for the previous store's acknowledgement: 128
    // store round trips per tile.)
    const bool lp_pairs = (reinterpret_cast<uintptr_t>(a.out_lp) & 3) == 0 && (a.ld_lp & 1) == 0;
    if (m0 + BM <= a.M && n0 + BN <= a.N && (MODE == 1 || lp_pairs) && a.ld_f32 < (int64_t(1) << 24) &&
        a.ld_lp < (int64_t(1) << 24)) {
        const int uw = __builtin_amdgcn_readfirstlane(wave);
        const int row0 = m0 + (uw / WGN) * WM, col0 = n0 + (uw % WGN) * WN;  // uniform
        const int half = lane >> 5, l31 = lane & 31, odd = lane & 1;
        typedef float f32x4_dword_aligned __attribute__((ext_vector_type(4), aligned(4)));
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            float inv[16];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                f32x4 g4 = {0.f, 0.f, 0.f, 0.f};
                if (a.g_rows != nullptr)
                    g4 = *reinterpret_cast<const f32x4_dword_aligned*>(a.g_rows + row0 + mb * 32 + q * 8 + half * 4);
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    inv[q * 4 + i] = a.g_rows != nullptr ? inv_b / pow2_scale(fabsf(g4[i]) * a.mult_a) : inv_common;
            }
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                float v[16];
                if constexpr (MODE != 0) {
                    float* blk = a.out_f32 + int64_t(row0 + mb * 32) * a.ld_f32 + (col0 + nb * 32);  // uniform
                    const uint32_t lane_off = uint32_t(half * 4) * uint32_t(a.ld_f32) + uint32_t(l31);
                    float prev[16];
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        prev[r] = a.first ? 0.f : blk[int64_t(((r >> 2) * 8 + (r & 3)) * a.ld_f32) + lane_off];
#pragma unroll
                    for (int r = 0; r < 16; ++r) v[r] = fmaf(acc[mb][nb][r], inv[r], prev[r]);
                    if constexpr (MODE == 1) {
#pragma unroll
                        for (int r = 0; r < 16; ++r) blk[int64_t(((r >> 2) * 8 + (r & 3)) * a.ld_f32) + lane_off] = v[r];
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 16; ++r) v[r] = acc[mb][nb][r] * inv[r];
                }
                if constexpr (MODE != 1) {
                    // 16-bit outputs: neighbouring lanes swap one value, the even lane then owns two columns of row
                    // r and the odd lane two columns of row r + 1 -- 4-byte stores, 64 contiguous bytes per row
                    typename E::type* blk = a.out_lp + int64_t(row0 + mb * 32) * a.ld_lp + (col0 + nb * 32);  // uniform
                    const uint32_t lane_off = uint32_t(half * 4 + odd) * uint32_t(a.ld_lp) + uint32_t(l31 & ~1);
#pragma unroll
                    for (int r = 0; r < 16; r += 2) {
                        const float give = odd ? v[r] : v[r + 1];
                        const float got = __builtin_bit_cast(
                            float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, give), 0xB1 /* quad_perm 1,0,3,2 */, 0xf, 0xf, true));
                        const uint32_t w = odd ? E::pack2(got, v[r + 1]) : E::pack2(v[r], got);
                        *reinterpret_cast<uint32_t*>(blk + int64_t(((r >> 2) * 8 + (r & 3)) * a.ld_lp) + lane_off) = w;
                    }
                }
            }
        }
        return;
    }
    // The running sum of a block is read as a whole before any of the block is written: with a load
    // and a store of the same array per element the compiler keeps them in program order, one memory
    // latency per element (67 us per tile instead of a few).
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        float inv[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = m0 + acc_row(wm, mb, r, lane);
            inv[r] = (a.g_rows != nullptr && row < a.M) ? inv_b / pow2_scale(fabsf(a.g_rows[row]) * a.mult_a) : inv_common;
        }
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int col = n0 + acc_col(wn, nb, lane);
            if (col >= a.N) continue;
            float prev[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + acc_row(wm, mb, r, lane);
                prev[r] = (MODE != 0 && !a.first && row < a.M) ? a.out_f32[int64_t(row) * a.ld_f32 + col] : 0.f;
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + acc_row(wm, mb, r, lane);
                if (row >= a.M) continue;
                const float v = fmaf(acc[mb][nb][r], inv[r], prev[r]);
                if (MODE == 1)
                    a.out_f32[int64_t(row) * a.ld_f32 + col] = v;
                else
                    E::store1(a.out_lp + int64_t(row) * a.ld_lp + col, v);
            }
        }
    }
}

// Two independent products in one launch: workgroups [0, grid_a) take `a` (epilogue MODE_A; its left operand is
// k-major), the rest take `b` (epilogue 0).  When the tile count of one product is not a multiple of the CU count, the other product's
// tiles fill the CUs its last round leaves idle.  grid_a is a multiple of 8 (the XCD mapping of `b` is kept).
template <int MODE_A, int ODT>
TRLK_HEAD_KERNEL void gemm_nt_pair_kernel(GemmArgs a, int grid_a, GemmArgs b) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    if (int(blockIdx.x) < grid_a)
        gemm_nt_body<TRLK_F16, MODE_A, ODT, true>(a, blockIdx.x, smem);
    else
        gemm_nt_body<TRLK_F16, 0, ODT>(b, int(blockIdx.x) - grid_a, smem);
}

// A single product (epilogue 1: fp32 output, overwritten or accumulated into).
template <int DT>
TRLK_HEAD_KERNEL void gemm_nt_kernel(GemmArgs a) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    gemm_nt_body<DT, 1, DT>(a, blockIdx.x, smem);
}

// fp32 [R, C] (row stride ld) -> bf16 [R, 6 * cpad] (row stride ldo, cpad = C rounded up to 8, padding zero): the three
// bf16 pieces x = p0 + p1 + p2 (p0 = bf16(x), p1 = bf16(x - p0), p2 = bf16(x - p0 - p1); 24 significant bits in all,
// with the exponent range of fp32) laid out along the contraction axis so that an NT product of an "A side" and a
// "B side" matrix sums the six piece products that matter, smallest first:
//   slot        0      1      2      3      4      5
//   A side      p2     p1     p0     p1     p0     p0
//   B side      p0     p1     p2     p0     p1     p0      (p1*p2, p2*p1, p2*p2 are below fp32 rounding: dropped)
__global__ __launch_bounds__(256) void split_bf16x3_kernel(const float* in, int64_t ld, int64_t R, int C, int cpad, int side,
                                                           uint16_t* out, int64_t ldo) {
    typedef Elem<TRLK_BF16> E;
    const int64_t r = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (r >= R || c >= cpad) return;
    float p[3] = {0.f, 0.f, 0.f};
    if (c < C) {
        const float x = in[r * ld + c];
        uint16_t h;
        E::store1(&h, x);
        p[0] = E::to_float(h);
        const float r1 = x - p[0];
        E::store1(&h, r1);
        p[1] = E::to_float(h);
        E::store1(&h, r1 - p[1]);
        p[2] = E::to_float(h);
    }
    const int a_map[6] = {2, 1, 0, 1, 0, 0}, b_map[6] = {0, 1, 2, 0, 1, 0};
    uint16_t* o = out + r * ldo + c;
#pragma unroll
    for (int sl = 0; sl < 6; ++sl) E::store1(o + int64_t(sl) * cpad, p[side == 0 ? a_map[sl] : b_map[sl]]);
}

// Largest magnitude of a bf16 [R, C8 * 8] matrix (row stride ld) as the bit pattern of that float, through an atomic
// maximum on `out` (non-negative floats order like unsigned integers; the caller clears `out`).
__global__ __launch_bounds__(256) void maxabs_bf16_kernel(const uint16_t* in, int64_t ld, int R, int C8, uint32_t* out) {
    uint32_t m = 0;
    auto take = [&](u32x4 q) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t lo = (q[i] << 16) & 0x7fff0000u, hi = q[i] & 0x7fff0000u;
            m = max(m, max(lo, hi));
        }
    };
    if (ld == int64_t(C8) * 8) {  // dense rows: one flat sweep, four loads in flight per lane
        const u32x4* p = reinterpret_cast<const u32x4*>(in);
        const int64_t n = int64_t(R) * C8, step = int64_t(gridDim.x) * 256;
        int64_t v = int64_t(blockIdx.x) * 256 + threadIdx.x;
        for (; v + 3 * step < n; v += 4 * step) {
            const u32x4 q0 = __builtin_nontemporal_load(p + v), q1 = __builtin_nontemporal_load(p + v + step),
                        q2 = __builtin_nontemporal_load(p + v + 2 * step), q3 = __builtin_nontemporal_load(p + v + 3 * step);
            take(q0), take(q1), take(q2), take(q3);
        }
        for (; v < n; v += step) take(__builtin_nontemporal_load(p + v));
    } else {
        for (int r = blockIdx.x; r < R; r += gridDim.x) {
            const u32x4* row = reinterpret_cast<const u32x4*>(in + int64_t(r) * ld);
            for (int c = threadIdx.x; c < C8; c += 256) take(row[c]);
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = max(m, uint32_t(__shfl_xor(int(m), off, 64)));
    if ((threadIdx.x & 63) == 0 && m != 0) atomicMax(out, m);
}
// The same for an fp32 vector.
__global__ __launch_bounds__(256) void maxabs_f32_kernel(const float* in, int64_t n, uint32_t* out) {
    uint32_t m = 0;
    for (int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x; i < n; i += int64_t(gridDim.x) * 256)
        m = max(m, __float_as_uint(in[i]) & 0x7fffffffu);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = max(m, uint32_t(__shfl_xor(int(m), off, 64)));
    if ((threadIdx.x & 63) == 0 && m != 0) atomicMax(out, m);
}

// [R, C] (ld) -> [C, ldo] with columns >= R zero-filled up to `fill`: 64 x 64 tiles through LDS.
// TO_F16: the input is bf16 and the output fp16, multiplied by the power of two that `in_max` (the input's largest
// magnitude) asks for.
// ROW_G: input row r is also multiplied by s_all / pow2_scale(|row_g[r]| * zs) (0 where row_g[r] is 0), s_all from
// `g_max`: what brings the columns of hidden^T into the scales of the d logits' columns (see above).
template <bool TO_F16, bool ROW_G = false>
__global__ __launch_bounds__(256) void transpose16_kernel(const uint16_t* in, int64_t ld, int R, int C, uint16_t* out,
                                                          int64_t ldo, int64_t fill, const uint32_t* in_max,
                                                          const float* row_g = nullptr, const uint32_t* g_max = nullptr,
                                                          float zs = 1.f) {
    // C, ld, ldo and fill are multiples of 8 and both matrices 16-byte aligned (the callers' operands are): a lane
    // moves 8 elements at a time.  Tile rows are skewed by 8 elements per group of 8 rows, which spreads the
    // 2-byte column reads of the second phase over all banks.
    constexpr int kStride = 136;
    __shared__ __attribute__((aligned(16))) uint16_t tile[64 * kStride];
    const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
    const int tid = threadIdx.x, hi = tid >> 3, lo = tid & 7;
    const float sc = TO_F16 ? slot_scale(in_max, 1.f) : 1.f;
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int row = hi + 32 * p, cc = lo * 8;
        u32x4 q = {0u, 0u, 0u, 0u};
        if (r0 + row < R && c0 + cc < C) q = *reinterpret_cast<const u32x4*>(in + int64_t(r0 + row) * ld + c0 + cc);
        if (TO_F16 || ROW_G) {
            float f = sc;
            if (ROW_G) {
                const float gr = r0 + row < R ? fabsf(row_g[r0 + row]) : 0.f;
                f = gr > 0.f ? sc * (slot_scale(g_max, zs) / pow2_scale(gr * zs)) : 0.f;
            }
            float x[8];
            if (TO_F16)
                Elem<TRLK_BF16>::unpack(q, x);
            else
                Elem<TRLK_F16>::unpack(q, x);
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] *= f;
            q = Elem<TRLK_F16>::pack(x);
        }
        *reinterpret_cast<u32x4*>(tile + row * kStride + cc + 8 * (row >> 3)) = q;
    }
    __syncthreads();
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int c = hi + 32 * p, r8 = lo;  // output row c0 + c, its columns r0 + 8 r8 .. + 7
        if (c0 + c < C && r0 + r8 * 8 < fill) {
            const uint16_t* src = tile + (r8 * 8) * kStride + c + 8 * r8;
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                w[i] = uint32_t(src[(2 * i) * kStride]) | (uint32_t(src[(2 * i + 1) * kStride]) << 16);
            const u32x4 q = {w[0], w[1], w[2], w[3]};
            *reinterpret_cast<u32x4*>(out + int64_t(c0 + c) * ldo + r0 + r8 * 8) = q;
        }
    }
}

int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

// d bias[v] = sum over tokens of dz[token, v]: row sums of the transposed dz copy (padding columns are zero).
__global__ __launch_bounds__(256) void dz_row_sum_kernel(const uint16_t* dzT, int64_t ld, int n_cols8, float* out,
                                                         const float* g, int n_tokens, float zs) {
    typedef Elem<TRLK_F16> E;
    const uint16_t* row = dzT + int64_t(blockIdx.x) * ld;
    float acc = 0.f;
    for (int c = threadIdx.x; c < n_cols8; c += 256) {
        const u32x4 w = *reinterpret_cast<const u32x4*>(row + c * 8);
        float x[8];
        E::unpack(w, x);
#pragma unroll
        for (int q = 0; q < 8; ++q) {  // column n is in token n's scale
            const int n = c * 8 + q;
            if (n < n_tokens) acc += x[q] / pow2_scale(fabsf(g[n]) * zs);
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    __shared__ float part[4];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) out[blockIdx.x] = part[0] + part[1] + part[2] + part[3];
}

// Row strides of the workspace matrices carry 128 extra bytes: their padded extents are multiples
// of large powers of two (tokens, chunk), and with such a stride the 256 rows of a tile step all
// fall into the same memory channels.
constexpr int64_t kLdSkew = 64;
struct BwdLayout {
    int64_t vpad, npad, cpad;    // padded extents (zero-filled)
    int64_t ld_v, ld_n, ld_c;    // row strides of [*, vpad], [*, npad], [*, cpad] matrices
    size_t off_wt, off_ht, off_dzt, off_dh, off_max, total;
    int64_t n_chunks;
};
BwdLayout bwd_layout(int64_t N, int64_t V, int64_t H, int64_t chunk) {
    BwdLayout l;
    l.vpad = round_up(V, BK);
    l.npad = round_up(N, BN);
    l.cpad = round_up(chunk < V ? chunk : V, BM);
    l.ld_v = l.vpad + kLdSkew;
    l.ld_n = l.npad + kLdSkew;
    l.ld_c = l.cpad + kLdSkew;
    size_t o = 0;
    auto take = [&](size_t bytes) {
        const size_t at = o;
        o += (bytes + 255) / 256 * 256;
        return at;
    };
    l.off_wt = take(size_t(H) * l.ld_c * 2);
    l.off_ht = take(size_t(H) * l.ld_n * 2);
    l.off_dzt = take(size_t(l.cpad) * l.ld_n * 2);
    l.off_dh = take(size_t(N) * H * 4);
    l.n_chunks = (V + l.cpad - 1) / l.cpad;
    l.off_max = take(size_t(2 + l.n_chunks) * 4);  // largest magnitudes: g, hidden, each chunk of W
    l.total = o;
    return l;
}

// Vocabulary splits of the forward.  A workgroup keeps one token block and walks over 1/splits of the
// vocabulary tiles, so the grid is token blocks x splits workgroups of equal length, one per CU at a
// time: the splits are chosen so that they fill whole rounds of the 256 CUs (65 token blocks x 8 splits
// would run 3 rounds for 2.03 rounds of work), preferring few splits.
constexpr int kCus = 256, kMinFwdSplits = 8, kMaxFwdSplits = 128;
int fwd_splits(int64_t n_tokens) {
    const int64_t n_tb = (n_tokens + BN - 1) / BN;
    int best = kMinFwdSplits;
    double best_cost = 1e30;
    for (int sp = kMinFwdSplits; sp <= kMaxFwdSplits; sp *= 2) {
        const double rounds = double(n_tb * sp) / kCus;
        const double cost = double((n_tb * sp + kCus - 1) / kCus) / rounds;
        if (cost < best_cost - 0.02) {  // more splits only for a gain of 2 % or more
            best_cost = cost;
            best = sp;
        }
    }
    return best;
}

int check_head(const char* what, const void* hidden, const void* weight, const int64_t* targets, int dtype, int64_t N,
               int64_t V, int64_t H, int64_t ldh, int64_t ldw, float temperature) {
    TRLK_REQUIRE(dtype == TRLK_BF16 || dtype == TRLK_F16, TRLK_ERR_BAD_DTYPE,
                 "%s: the fused head takes bf16 or fp16 operands (dtype code %d)", what, dtype);
    TRLK_REQUIRE(N >= 0 && V >= 1 && H >= 1, TRLK_ERR_BAD_SHAPE, "%s: bad sizes N=%lld V=%lld H=%lld", what, (long long)N,
                 (long long)V, (long long)H);
    TRLK_REQUIRE(N < (int64_t(1) << 31) - BN && V < (int64_t(1) << 31) - BM, TRLK_ERR_BAD_SHAPE, "%s: N or V too large",
                 what);
    TRLK_REQUIRE(H % 8 == 0 && ldh % 8 == 0 && ldw % 8 == 0 && ldh >= H && ldw >= H, TRLK_ERR_BAD_STRIDE,
                 "%s: H and the row strides must be multiples of 8 elements (H=%lld ldh=%lld ldw=%lld)", what,
                 (long long)H, (long long)ldh, (long long)ldw);
    TRLK_REQUIRE(temperature > 0.f && temperature < INFINITY, TRLK_ERR_BAD_VALUE, "%s: temperature must be positive", what);
    if (N > 0) {
        TRLK_REQUIRE(hidden && weight && targets, TRLK_ERR_NULL_POINTER, "%s: null operand pointer", what);
        TRLK_REQUIRE(reinterpret_cast<uintptr_t>(hidden) % 16 == 0 && reinterpret_cast<uintptr_t>(weight) % 16 == 0,
                     TRLK_ERR_BAD_STRIDE, "%s: operands must be 16-byte aligned", what);
    }
    return TRLK_OK;
}

template <typename Kern>
int reserve_head_lds(Kern kern, const char* what);

template <typename Kern>
int launch_head_pair(Kern kern, int grid_a, const GemmArgs& a, int grid_b, const GemmArgs& b, hipStream_t s,
                     const char* what) {
    if (int rc = reserve_head_lds(kern, what)) return rc;
    hipLaunchKernelGGL(kern, dim3(grid_a + grid_b), dim3(kHeadThreads), kHeadLdsBytes, s, a, grid_a, b);
    return launch_status(what);
}

template <typename Kern, typename Args>
int launch_head(Kern kern, int grid, const Args& a, hipStream_t s, const char* what) {
    if (int rc = reserve_head_lds(kern, what)) return rc;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kHeadThreads), kHeadLdsBytes, s, a);
    return launch_status(what);
}

template <typename Kern>
int reserve_head_lds(Kern kern, const char* what) {
    // dynamic LDS above 64 KiB has to be allowed per kernel and device once
    struct Done {
        const void* kern;
        int device;
    };
    static thread_local Done configured[32] = {};
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) device = 0;
    const void* key = reinterpret_cast<const void*>(kern);
    for (const Done& c : configured)
        if (c.kern == key && c.device == device) return TRLK_OK;
    const hipError_t e = hipFuncSetAttribute(key, hipFuncAttributeMaxDynamicSharedMemorySize, kHeadLdsBytes);
    if (e != hipSuccess) return fail(int(e), "%s: cannot reserve %d bytes of LDS: %s", what, kHeadLdsBytes, hipGetErrorString(e));
    for (Done& c : configured)
        if (c.kern == nullptr) {
            c.kern = key;
            c.device = device;
            break;
        }
    return TRLK_OK;
}

}  // namespace
}  // namespace trlk

using namespace trlk;

extern "C" size_t trlk_fused_head_fwd_workspace_bytes(int64_t n_tokens) {
    return n_tokens > 0 ? size_t(n_tokens) * (fwd_splits(n_tokens) * 4 + 1) * sizeof(float) : 0;
}

extern "C" size_t trlk_fused_head_stash_bytes(int64_t n_tokens, int64_t vocab, int64_t* out_ld) {
    if (n_tokens <= 0 || vocab <= 0) return 0;
    const int64_t ld = round_up(n_tokens, BN);
    if (out_ld) *out_ld = ld;
    return size_t(StashView::rows8(round_up(vocab, BM))) * size_t(ld) * 8;
}

extern "C" size_t trlk_fused_head_bwd_workspace_bytes(int64_t n_tokens, int64_t vocab, int64_t hidden_size,
                                                      int64_t chunk_size) {
    if (n_tokens <= 0 || vocab <= 0 || hidden_size <= 0 || chunk_size <= 0) return 0;
    return bwd_layout(n_tokens, vocab, hidden_size, chunk_size).total;
}

extern "C" int trlk_fused_head_fwd(const void* d_hidden, const void* d_weight, const int64_t* d_targets, int dtype,
                                   int64_t n_tokens, int64_t vocab, int64_t hidden_size, int64_t hidden_stride,
                                   int64_t weight_stride, float temperature, float final_logit_softcapping,
                                   float logit_scale, const float* d_bias, float* d_out_logp, float* d_out_entropy,
                                   float* d_out_log_z, float* d_out_target_is_max, void* d_out_stash,
                                   int64_t stash_ld, int32_t* d_error_flag, void* d_workspace, size_t workspace_bytes,
                                   trlk_stream_t stream) {
    clear_error();
    if (int rc = check_head("fused_head_fwd", d_hidden, d_weight, d_targets, dtype, n_tokens, vocab, hidden_size,
                            hidden_stride, weight_stride, temperature))
        return rc;
    if (n_tokens == 0) return TRLK_OK;
    TRLK_REQUIRE(d_out_logp && d_out_entropy && d_out_log_z, TRLK_ERR_NULL_POINTER, "fused_head_fwd: null output pointer");
    TRLK_REQUIRE(d_workspace && workspace_bytes >= trlk_fused_head_fwd_workspace_bytes(n_tokens), TRLK_ERR_WORKSPACE,
                 "fused_head_fwd: workspace of %zu bytes needed, %zu given", trlk_fused_head_fwd_workspace_bytes(n_tokens),
                 workspace_bytes);
    TRLK_REQUIRE(d_out_stash == nullptr || (stash_ld >= round_up(n_tokens, BN) && stash_ld % 4 == 0 &&
                                            stash_ld < (int64_t(1) << 31) / 16 &&
                                            reinterpret_cast<uintptr_t>(d_out_stash) % 16 == 0),
                 TRLK_ERR_BAD_STRIDE, "fused_head_fwd: the stash needs a 16-byte aligned buffer with a row stride >= %lld (got %lld)",
                 (long long)round_up(n_tokens, BN), (long long)stash_ld);
    hipStream_t s = static_cast<hipStream_t>(stream);
    HeadArgs a{};
    a.hidden = static_cast<const uint16_t*>(d_hidden);
    a.weight = static_cast<const uint16_t*>(d_weight);
    a.targets = d_targets;
    a.bias = d_bias;
    a.stash = StashView{static_cast<char*>(d_out_stash), stash_ld, round_up(vocab, BM)};
    a.N = int(n_tokens);
    a.V = int(vocab);
    a.H = int(hidden_size);
    a.ldh = hidden_stride;
    a.ldw = weight_stride;
    a.logit_scale = logit_scale;
    a.inv_t = 1.f / temperature;
    a.softcap = final_logit_softcapping > 0.f ? final_logit_softcapping : 0.f;
    const int n_vt = int((vocab + BM - 1) / BM);
    int splits = fwd_splits(n_tokens);  // what the workspace was sized for
    while (splits > 1 && n_vt < 4 * splits) splits /= 2;  // at least 4 vocabulary tiles per workgroup
    a.v_splits = splits;
    a.tiles_per_split = (n_vt + splits - 1) / splits;
    a.partial = static_cast<float*>(d_workspace);
    a.tgt = a.partial + size_t(n_tokens) * splits * 4;
    hipLaunchKernelGGL(head_fill_kernel, dim3(unsigned((n_tokens + 255) / 256)), dim3(256), 0, s, a.tgt, n_tokens, NAN);
    if (int rc = launch_status("fused_head_fwd (fill)")) return rc;
    const int n_tb = int((n_tokens + BN - 1) / BN);
    const int grid = xcd_patch_grid(n_tb, splits);
    const char* what = "fused_head_fwd";
    int rc;
    const bool general = a.softcap > 0.f || !(a.logit_scale * a.inv_t > 0.f);
    const bool staged = hidden_size % TRLK_HEAD_BK_FWD != 0;
    auto launch_fwd = [&](auto stash_tag, auto general_tag) {
        constexpr bool kS = decltype(stash_tag)::value, kG = decltype(general_tag)::value;
        if (staged)
            return dtype == TRLK_BF16 ? launch_head(fused_head_fwd_kernel<TRLK_BF16, kS, kG, true>, grid, a, s, what)
                                      : launch_head(fused_head_fwd_kernel<TRLK_F16, kS, kG, true>, grid, a, s, what);
        return dtype == TRLK_BF16 ? launch_head(fused_head_fwd_kernel<TRLK_BF16, kS, kG, false>, grid, a, s, what)
                                  : launch_head(fused_head_fwd_kernel<TRLK_F16, kS, kG, false>, grid, a, s, what);
    };
    if (d_out_stash != nullptr)
        rc = general ? launch_fwd(std::true_type{}, std::true_type{}) : launch_fwd(std::true_type{}, std::false_type{});
    else
        rc = general ? launch_fwd(std::false_type{}, std::true_type{}) : launch_fwd(std::false_type{}, std::false_type{});
    if (rc) return rc;
    hipLaunchKernelGGL(head_merge_kernel, dim3(unsigned((n_tokens + 255) / 256)), dim3(256), 0, s, a.partial, a.tgt,
                       d_targets, int(n_tokens), int(vocab), splits, d_out_logp, d_out_entropy, d_out_log_z,
                       d_out_target_is_max, d_error_flag, d_out_stash != nullptr ? a.stash.zt() : nullptr);
    return launch_status("fused_head_fwd (merge)");
}

extern "C" int trlk_fused_head_bwd(const void* d_hidden, const void* d_weight, const int64_t* d_targets, int dtype,
                                   int64_t n_tokens, int64_t vocab, int64_t hidden_size, int64_t hidden_stride,
                                   int64_t weight_stride, float temperature, float final_logit_softcapping,
                                   float logit_scale, const float* d_bias, const float* d_log_z, const float* d_g_logp,
                                   int64_t chunk_size, const void* d_stash, int64_t stash_ld, const int32_t* d_stash_cols,
                                   void* d_out_dhidden, void* d_out_dweight, float* d_out_dbias, void* d_workspace,
                                   size_t workspace_bytes, trlk_stream_t stream) {
    clear_error();
    if (int rc = check_head("fused_head_bwd", d_hidden, d_weight, d_targets, dtype, n_tokens, vocab, hidden_size,
                            hidden_stride, weight_stride, temperature))
        return rc;
    TRLK_REQUIRE(chunk_size >= 1, TRLK_ERR_BAD_VALUE, "fused_head_bwd: chunk_size must be >= 1");
    TRLK_REQUIRE(d_out_dhidden && d_out_dweight, TRLK_ERR_NULL_POINTER, "fused_head_bwd: null output pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (n_tokens == 0) {  // no tokens: both gradients are zero
        hipLaunchKernelGGL(head_fill_kernel, dim3(unsigned((vocab * hidden_size / 2 + 255) / 256)), dim3(256), 0, s,
                           static_cast<float*>(d_out_dweight), vocab * hidden_size / 2, 0.f);
        if (d_out_dbias)
            hipLaunchKernelGGL(head_fill_kernel, dim3(unsigned((vocab + 255) / 256)), dim3(256), 0, s, d_out_dbias, vocab, 0.f);
        return launch_status("fused_head_bwd (zero dW)");
    }
    TRLK_REQUIRE(d_log_z && d_g_logp, TRLK_ERR_NULL_POINTER, "fused_head_bwd: log_z / g_logp pointer is null");
    TRLK_REQUIRE(d_stash == nullptr || chunk_size <= int64_t(65535) * kSdzRows || vocab <= int64_t(65535) * kSdzRows,
                 TRLK_ERR_BAD_SHAPE, "fused_head_bwd: chunk of %lld rows is too large for the stash path",
                 (long long)chunk_size);
    TRLK_REQUIRE(d_stash_cols == nullptr || d_stash != nullptr, TRLK_ERR_NULL_POINTER,
                 "fused_head_bwd: stash columns given without a stash");
    TRLK_REQUIRE(d_stash == nullptr || ((d_stash_cols != nullptr || stash_ld >= round_up(n_tokens, BN)) && stash_ld % 4 == 0 &&
                                        reinterpret_cast<uintptr_t>(d_stash) % 16 == 0),
                 TRLK_ERR_BAD_STRIDE, "fused_head_bwd: the stash needs a 16-byte aligned buffer with a row stride >= %lld (got %lld)",
                 (long long)round_up(n_tokens, BN), (long long)stash_ld);
    const int64_t chunk = round_up(chunk_size < vocab ? chunk_size : vocab, BM);
    const BwdLayout l = bwd_layout(n_tokens, vocab, hidden_size, chunk);
    TRLK_REQUIRE(d_workspace && workspace_bytes >= l.total, TRLK_ERR_WORKSPACE,
                 "fused_head_bwd: workspace of %zu bytes needed, %zu given", l.total, workspace_bytes);
    char* ws = static_cast<char*>(d_workspace);
    uint16_t* wt = reinterpret_cast<uint16_t*>(ws + l.off_wt);    // [H, cpad], row stride ld_c (one chunk at a time)
    uint16_t* ht = reinterpret_cast<uint16_t*>(ws + l.off_ht);    // [H, npad], row stride ld_n
    uint16_t* dzt = reinterpret_cast<uint16_t*>(ws + l.off_dzt);  // [cpad, npad], row stride ld_n
    float* dh = reinterpret_cast<float*>(ws + l.off_dh);          // [N, H]
    uint32_t* maxima = reinterpret_cast<uint32_t*>(ws + l.off_max);  // [0] g, [1] hidden, [2] W
    const int H = int(hidden_size), N = int(n_tokens), V = int(vocab);
    const bool from_bf16 = dtype == TRLK_BF16;  // the products' operands are fp16: bf16 inputs are converted on the way
    const uint32_t* max_g = maxima;
    const uint32_t* max_h = from_bf16 ? maxima + 1 : nullptr;
    hipLaunchKernelGGL(head_fill_kernel, dim3(unsigned((2 + l.n_chunks + 255) / 256)), dim3(256), 0, s,
                       reinterpret_cast<float*>(maxima), 2 + l.n_chunks, 0.f);
    hipLaunchKernelGGL(maxabs_f32_kernel, dim3(unsigned(N < 65536 ? (N + 255) / 256 : 256)), dim3(256), 0, s, d_g_logp,
                       n_tokens, maxima);
    if (from_bf16) {
        hipLaunchKernelGGL(maxabs_bf16_kernel, dim3(unsigned(N < 2048 ? N : 2048)), dim3(256), 0, s,
                           static_cast<const uint16_t*>(d_hidden), hidden_stride, N, H / 8, maxima + 1);
        // one scale for the whole weight: a single sweep over it instead of one per chunk
        hipLaunchKernelGGL(maxabs_bf16_kernel, dim3(unsigned(V < 4096 ? V : 4096)), dim3(256), 0, s,
                           static_cast<const uint16_t*>(d_weight), weight_stride, V, H / 8, maxima + 2);
        hipLaunchKernelGGL((transpose16_kernel<true, true>), dim3((H + 63) / 64, unsigned((l.npad + 63) / 64)), dim3(256), 0, s,
                           static_cast<const uint16_t*>(d_hidden), hidden_stride, N, H, ht, l.ld_n, l.npad, max_h, d_g_logp,
                           max_g, logit_scale / temperature);
    } else {
        hipLaunchKernelGGL((transpose16_kernel<false, true>), dim3((H + 63) / 64, unsigned((l.npad + 63) / 64)), dim3(256), 0, s,
                           static_cast<const uint16_t*>(d_hidden), hidden_stride, N, H, ht, l.ld_n, l.npad, max_h, d_g_logp,
                           max_g, logit_scale / temperature);
    }
    if (int rc = launch_status("fused_head_bwd (hidden^T)")) return rc;

    HeadArgs a{};
    a.hidden = static_cast<const uint16_t*>(d_hidden);
    a.weight = static_cast<const uint16_t*>(d_weight);
    a.targets = d_targets;
    a.bias = d_bias;
    a.N = N;
    a.V = V;
    a.H = H;
    a.ldh = hidden_stride;
    a.ldw = weight_stride;
    a.logit_scale = logit_scale;
    a.inv_t = 1.f / temperature;
    a.softcap = final_logit_softcapping > 0.f ? final_logit_softcapping : 0.f;
    a.log_z = d_log_z;
    a.g = d_g_logp;
    a.stash = StashView{static_cast<char*>(const_cast<void*>(d_stash)), stash_ld, round_up(vocab, BM)};
    a.stash_cols = d_stash_cols;
    a.dzT = dzt;
    a.ldzt = l.ld_n;
    a.g_max = max_g;
    const float zs = logit_scale / temperature;  // |dz[n, v]| <= |g[n]| * zs
    const int n_tb = int((n_tokens + BN - 1) / BN);
    const int n_ht = (H + BN - 1) / BN;
    for (int64_t c0 = 0; c0 < vocab; c0 += chunk) {
        const int64_t c1 = c0 + chunk < vocab ? c0 + chunk : vocab;
        const int rows = int(c1 - c0);
        const int kpad = int(round_up(rows, BM));  // dz / dz^T are zero beyond the chunk's rows
        a.c0 = int(c0);
        a.c1 = int(c1);
        const int n_vt = (rows + BM - 1) / BM;
        int rc;
        if (d_stash != nullptr) {
            a.sdz_token_blocks = int(l.npad / kSdzTokens);
            a.sdz_tiles = a.sdz_token_blocks * int(kpad / kSdzRows);
            const dim3 grid(unsigned((a.sdz_tiles + 7) / 8 * 8));
            const bool capped = a.softcap > 0.f;
            if (d_stash_cols && capped)
                hipLaunchKernelGGL((head_dz_from_stash_kernel<true, true>), grid, dim3(256), 0, s, a);
            else if (d_stash_cols)
                hipLaunchKernelGGL((head_dz_from_stash_kernel<true, false>), grid, dim3(256), 0, s, a);
            else if (capped)
                hipLaunchKernelGGL((head_dz_from_stash_kernel<false, true>), grid, dim3(256), 0, s, a);
            else
                hipLaunchKernelGGL((head_dz_from_stash_kernel<false, false>), grid, dim3(256), 0, s, a);
            rc = launch_status("fused_head_bwd (dz from the stash)");
        } else {
            rc = dtype == TRLK_BF16
                     ? launch_head(fused_head_dz_kernel<TRLK_BF16>, xcd_patch_grid(n_tb, n_vt), a, s, "fused_head_bwd (dz)")
                     : launch_head(fused_head_dz_kernel<TRLK_F16>, xcd_patch_grid(n_tb, n_vt), a, s, "fused_head_bwd (dz)");
        }
        if (rc) return rc;
        if (d_out_dbias) {
            hipLaunchKernelGGL(dz_row_sum_kernel, dim3(rows), dim3(256), 0, s, dzt, l.ld_n, int(l.npad / 8), d_out_dbias + c0,
                               d_g_logp, N, zs);
            if (int rc2 = launch_status("fused_head_bwd (dBias)")) return rc2;
        }
        const bool first = c0 == 0, last = c1 == vocab;
        // W_chunk^T [H, kpad] (columns beyond the chunk's rows are zero): the chunk's own transposed copy keeps the
        // row stride of this operand as short as that of the other three
        const uint16_t* w_chunk = static_cast<const uint16_t*>(d_weight) + c0 * weight_stride;
        const uint32_t* max_w = from_bf16 ? maxima + 2 : nullptr;
        const dim3 tgrid((H + 63) / 64, unsigned((kpad + 63) / 64));
        if (from_bf16) {
            hipLaunchKernelGGL(transpose16_kernel<true>, tgrid, dim3(256), 0, s, w_chunk, weight_stride, rows, H, wt, l.ld_c,
                               int64_t(kpad), max_w);
        } else {
            hipLaunchKernelGGL(transpose16_kernel<false>, tgrid, dim3(256), 0, s, w_chunk, weight_stride, rows, H, wt, l.ld_c,
                               int64_t(kpad), max_w);
        }
        if (int rc2 = launch_status("fused_head_bwd (W^T)")) return rc2;
        // dHidden[N, H] += dz[N, chunk] * (W_chunk^T[H, chunk])^T
        GemmArgs gh{};
        gh.A = Operand{dzt, l.ld_n, N};  // k-major: [chunk rows, tokens]
        gh.B = Operand{wt, l.ld_c, H};
        gh.M = N;
        gh.N = H;
        gh.K = kpad;
        gh.out_f32 = dh;
        gh.ld_f32 = H;
        gh.out_lp = static_cast<uint16_t*>(d_out_dhidden);
        gh.ld_lp = H;
        gh.first = first;
        gh.max_a = nullptr;  // the rows of dz carry their own scales
        gh.g_rows = d_g_logp;
        gh.mult_a = zs;
        gh.max_b = max_w;
        const int ghgrid = xcd_patch_grid(n_tb, n_ht);
        // dW[chunk, H] = dz^T[chunk, N] * (hidden^T[H, N])^T
        GemmArgs gw{};
        gw.A = Operand{dzt, l.ld_n, kpad};
        gw.B = Operand{ht, l.ld_n, H};
        gw.M = rows;
        gw.N = H;
        gw.K = int(l.npad);
        gw.out_lp = static_cast<uint16_t*>(d_out_dweight) + c0 * hidden_size;
        gw.ld_lp = hidden_size;
        gw.first = 1;
        gw.max_a = max_g;
        gw.g_rows = nullptr;
        gw.mult_a = zs;
        gw.max_b = max_h;
        // both products of the chunk in one launch (dHidden's workgroups first)
        const int gwgrid = xcd_patch_grid(n_vt, n_ht);
        const char* what = "fused_head_bwd (dHidden, dW)";
        if (last)
            rc = from_bf16 ? launch_head_pair(gemm_nt_pair_kernel<2, TRLK_BF16>, ghgrid, gh, gwgrid, gw, s, what)
                           : launch_head_pair(gemm_nt_pair_kernel<2, TRLK_F16>, ghgrid, gh, gwgrid, gw, s, what);
        else
            rc = from_bf16 ? launch_head_pair(gemm_nt_pair_kernel<1, TRLK_BF16>, ghgrid, gh, gwgrid, gw, s, what)
                           : launch_head_pair(gemm_nt_pair_kernel<1, TRLK_F16>, ghgrid, gh, gwgrid, gw, s, what);
        if (rc) return rc;
    }
    return TRLK_OK;
}

extern "C" int trlk_split_bf16x3(const float* d_in, int64_t rows, int64_t cols, int64_t ld_in, int side, void* d_out,
                                 int64_t ld_out, trlk_stream_t stream) {
    clear_error();
    TRLK_REQUIRE(rows >= 0 && cols >= 1 && cols < (int64_t(1) << 28), TRLK_ERR_BAD_SHAPE, "split_bf16x3: bad shape %lld x %lld",
                 (long long)rows, (long long)cols);
    TRLK_REQUIRE(side == 0 || side == 1, TRLK_ERR_BAD_VALUE, "split_bf16x3: side must be 0 (A) or 1 (B), got %d", side);
    const int64_t cpad = round_up(cols, 8);
    TRLK_REQUIRE(ld_in >= cols && ld_out >= 6 * cpad && ld_out % 8 == 0, TRLK_ERR_BAD_STRIDE,
                 "split_bf16x3: row strides too short (in %lld for %lld columns, out %lld for %lld)", (long long)ld_in,
                 (long long)cols, (long long)ld_out, (long long)(6 * cpad));
    if (rows == 0) return TRLK_OK;
    TRLK_REQUIRE(d_in && d_out, TRLK_ERR_NULL_POINTER, "split_bf16x3: null pointer");
    TRLK_REQUIRE(rows < 65536 * int64_t(32768), TRLK_ERR_BAD_SHAPE, "split_bf16x3: too many rows");
    hipStream_t s = static_cast<hipStream_t>(stream);
    for (int64_t r0 = 0; r0 < rows; r0 += 65535) {  // grid.y limit
        const int64_t nr = rows - r0 < 65535 ? rows - r0 : 65535;
        hipLaunchKernelGGL(split_bf16x3_kernel, dim3(unsigned((cpad + 255) / 256), unsigned(nr)), dim3(256), 0, s,
                           d_in + r0 * ld_in, ld_in, nr, int(cols), int(cpad), side,
                           static_cast<uint16_t*>(d_out) + r0 * ld_out, ld_out);
    }
    return launch_status("split_bf16x3");
}

extern "C" int trlk_gemm_nt(const void* d_a, int64_t lda, const void* d_b, int64_t ldb, int dtype, int64_t m, int64_t n,
                            int64_t k, float* d_out, int64_t ldo, int accumulate, trlk_stream_t stream) {
    clear_error();
    TRLK_REQUIRE(dtype == TRLK_BF16 || dtype == TRLK_F16, TRLK_ERR_BAD_DTYPE, "gemm_nt: bf16 or fp16 operands (dtype code %d)",
                 dtype);
    TRLK_REQUIRE(m >= 0 && n >= 0 && k >= 8 && m < (int64_t(1) << 31) - BM && n < (int64_t(1) << 31) - BN &&
                     k < (int64_t(1) << 31) - BK,
                 TRLK_ERR_BAD_SHAPE, "gemm_nt: bad sizes m=%lld n=%lld k=%lld", (long long)m, (long long)n, (long long)k);
    TRLK_REQUIRE(k % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0 && lda >= k && ldb >= k && ldo >= n, TRLK_ERR_BAD_STRIDE,
                 "gemm_nt: k and the operands' row strides must be multiples of 8 elements (k=%lld lda=%lld ldb=%lld ldo=%lld)",
                 (long long)k, (long long)lda, (long long)ldb, (long long)ldo);
    // tile-relative operand offsets are 32-bit
    TRLK_REQUIRE(lda * 2 * BM < (int64_t(1) << 32) && ldb * 2 * BN < (int64_t(1) << 32), TRLK_ERR_BAD_STRIDE,
                 "gemm_nt: row strides too long (lda=%lld ldb=%lld)", (long long)lda, (long long)ldb);
    if (m == 0 || n == 0) return TRLK_OK;
    TRLK_REQUIRE(d_a && d_b && d_out, TRLK_ERR_NULL_POINTER, "gemm_nt: null pointer");
    TRLK_REQUIRE(reinterpret_cast<uintptr_t>(d_a) % 16 == 0 && reinterpret_cast<uintptr_t>(d_b) % 16 == 0, TRLK_ERR_BAD_STRIDE,
                 "gemm_nt: operands must be 16-byte aligned");
    GemmArgs g{};
    g.A = Operand{static_cast<const uint16_t*>(d_a), lda, int(m)};
    g.B = Operand{static_cast<const uint16_t*>(d_b), ldb, int(n)};
    g.M = int(m);
    g.N = int(n);
    g.K = int(k);
    g.out_f32 = d_out;
    g.ld_f32 = ldo;
    g.first = accumulate ? 0 : 1;
    g.mult_a = 1.f;
    const int grid = xcd_patch_grid(int((m + BM - 1) / BM), int((n + BN - 1) / BN));
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dtype == TRLK_BF16 ? launch_head(gemm_nt_kernel<TRLK_BF16>, grid, g, s, "gemm_nt")
                              : launch_head(gemm_nt_kernel<TRLK_F16>, grid, g, s, "gemm_nt");
}
