// K7: from the logits straight to the GRPO loss gradient, one read and one write of the logits-sized data.
//
// The two-pass path reads the logits twice (K1 for the log-probs, K3 for the gradient) because the loss sits
// between them.  For the token-level GRPO losses the gradient coefficient of a token depends only on that
// token's own log-prob, on per-token inputs (old / reference log-probs, advantage, mask, weight) and on
// normalisers that are known from the mask before any logit is read.  A 1024-lane workgroup can hold a whole
// vocabulary row of logits in registers (up to kMaxVec 16-byte vectors per lane: 8 16-bit or 4 fp32 logits each), so one workgroup
// per row loads the row once, reduces it to (lse, entropy, target logit), evaluates the token's loss terms
// with the same device functions as the [B, T]-sized loss kernel, and writes the row's dlogits from the
// registers.  Rows outside the completion mask are never read: their gradient row is zero-filled and their
// outputs are 0.
#include <mutex>
#include <vector>

#include "common.hpp"
#include "grpo_token.hpp"

namespace trlk {
namespace {

constexpr int kFThreads = 1024;
constexpr int kFWaves = kFThreads / kWave;
constexpr int kMaxVec = 20;  // 16-byte vectors of a row per lane in registers: rows of up to 20 * 1024 * 8 = 163840 logits
constexpr int kVecStep = 4;  // the kernel is built for 4, 8, ... kMaxVec vectors per lane; the host picks the smallest that holds the row
// Longer rows keep what the registers cannot hold in the CU's LDS: up to kMaxLdsVec more vectors per lane (16 KiB of
// LDS each; 9 of them leave room for the reduction scratch in the 160 KiB), in builds of kLdsStep: rows of up to
// 29 * 1024 * 8 = 237568 logits.
constexpr int kMaxLdsVec = 9, kLdsStep = 3;
// Rows longer still (the 256000- and 262144-entry vocabularies) read their last vectors twice: once ahead of the row
// for the sums, once after it for the gradient, by which time the workgroup has read them so recently that they
// come from the L2.  Up to kMaxExtraVec such vectors per lane: rows of up to 41 * 1024 * 8 = 335872 16-bit logits
// (half as many fp32 ones).
constexpr int kMaxExtraVec = 12;  // (37 on-chip + extra vectors x 1024 x 4 fp32 logits covers the 151936-entry rows in fp32 too)
constexpr int kWideVec = kMaxVec;  // register vectors of the builds with vectors in LDS

typedef __attribute__((address_space(1))) const u32x4 GlobalVecIn;
typedef __attribute__((address_space(1))) u32x4 GlobalVecOut;
typedef u32x4 u32x4_u __attribute__((aligned(2)));  // a 16-byte vector at any element alignment
typedef __attribute__((address_space(1))) u32x4_u GlobalVecOutU;

struct FusedArgs {
    const void* logits;
    int64_t rows_per_seq, vocab, seq_stride, row_stride;
    const int64_t* index;  // [n_seq * rows_per_seq]
    float temperature;
    const float *old_logp, *ref_logp, *adv, *mask, *token_weight, *row_scale, *seq_coef;
    const float* ent_weight;  // [rows] d loss / d entropy of the token, already normalised, or null
    int64_t adv_stride_b, adv_stride_t;
    int policy_term;
    float eps_low, eps_high, delta, beta;
    int bias_kl;
    float sapo_tau_pos, sapo_tau_neg;
    float *out_logp, *out_entropy, *out_lse;
    void* dlogits;
    int64_t out_rows_per_seq, out_row_offset, out_seq_stride, out_row_stride;
    int32_t* error_flag;
    int64_t total_rows;  // output rows: the grid is rounded up to a multiple of 8
    int all_rows;  // also read the rows with mask == 0 for their log-prob and entropy (their gradient is zero either way)
};

// One 1 KiB transfer from memory straight into LDS: 16 bytes per lane from `src` to LDS address `lds` + 16 * lane
// (`lds` uniform over the wave).  (m0 is a reserved register; naming it as clobbered keeps the compiler's values out.)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void lds_transfer(const u32x4* src, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds),
                 "v"(reinterpret_cast<uint64_t>(src))
                 : "memory", "m0");
}
#pragma clang diagnostic pop

// One workgroup of 1024 lanes per output row; NVEC = 16-byte vectors of the row a lane holds (the last kVecStep of
// them may lie beyond the row's end for some lanes).  A workgroup fills its CU's register file, so nothing else
// runs beside it: the arithmetic has to overlap the row's own memory traffic.  Hence
//   * the per-row scalars are loaded first, from uniform addresses before any store: scalar loads, which return
//     long before (and independently of) the row's vector loads; the target's logit is requested right behind the row;
//   * the exponentials are summed while the row arrives: a lane takes its reference exponent r0 from its FIRST
//     vector (an integer, so bringing the lanes' sums to a common exponent afterwards is exact) and consumes each
//     vector as its load retires.  Later logits may exceed the first vector's by 128 / (log2(e) / T) before a
//     term overflows; a row where that happens (or one that holds inf / NaN) is detected by its non-finite sums
//     and takes the exact two-sweep reduction over the registers instead.
//   * NLDS > 0 (rows too long for the registers): vectors NVEC ... NVEC + NLDS - 1 of a lane travel from memory straight
//     into LDS, 1 KiB per wave and transfer, issued before the register loads; a lane only ever reads back the 16
//     bytes its own transfer wrote, so the wave's own wait for its transfers is all the synchronisation they need.
//   * EXTRA (rows too long for registers and LDS together): the vectors beyond are summed before the row proper is
//     requested (four loads in flight; their registers are free again when the row's loads go out) and read again at
//     the end for their gradient.
//   * RAGGED (rows that are not whole aligned vectors: a vocabulary that is no multiple of the vector width): the
//     row is taken in aligned vectors from its first 16-byte boundary on; the up to EPV - 1 elements before that and
//     after the last whole vector belong to one lane each, which reads its element ahead of the row for the sums
//     and again after the row's stores for its gradient.  The gradient row may sit at another alignment than the
//     logits row: its vectors are stored through accesses that need none.
template <int DT, int NVEC, int NLDS, bool EXTRA = false, bool RAGGED = false>
__global__ __launch_bounds__(kFThreads) void grpo_fused_kernel(FusedArgs a) {
    typedef Elem<DT> E;
    typedef typename E::type T;
    constexpr int EPV = E::EPV;
    // (the last register vectors keep their end-of-row test in the builds with vectors in LDS too, where it is always
    // true: without it the compiler unpacks every register vector ahead of its use and spills a hundred registers)
    constexpr int kTail = NVEC - kVecStep;
    extern __shared__ __attribute__((aligned(16))) char overflow[];  // [NLDS][1024 lanes] 16-byte vectors
    __shared__ float red[7][kFWaves];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    // The hardware deals consecutive workgroups to the eight XCDs in turn.  Each XCD takes one contiguous eighth of
    // the rows and walks it in order, instead of every eighth row of the whole tensor: eight separate streams of reads
    // and writes, one per XCD.  Measured on bf16 [64, 1024, 151936] with the benchmark's mask: 5.65 -> 5.24 ms
    // (every row read: 7.25 -> 6.86 ms; every row active: 7.55 -> 7.28 ms).
    const int64_t per_xcd = int64_t(gridDim.x) >> 3;  // (the grid is a multiple of 8)
    const int64_t orow = int64_t(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (orow >= a.total_rows) return;
    const int64_t b = orow / a.out_rows_per_seq;
    const int64_t to = orow - b * a.out_rows_per_seq;
    const int64_t t = to - a.out_row_offset;
    const bool inside = t >= 0 && t < a.rows_per_seq;
    const int64_t row = b * a.rows_per_seq + (inside ? t : 0);
    int nv = int(a.vocab / EPV);  // whole vectors of the row (RAGGED: counted from its first 16-byte boundary, set below)
    float m = 0.f, A = 0.f, old_lp = 0.f, ref_lp = 0.f, w = 1.f, coef = 0.f, scale = 0.f, h = 0.f;
    int64_t idx = -1;
    if (inside) {
        m = a.mask[row];
        idx = a.index[row];
        A = a.adv[b * a.adv_stride_b + t * a.adv_stride_t];
        if (a.old_logp) old_lp = a.old_logp[row];
        if (a.beta != 0.f) ref_lp = a.ref_logp[row];
        if (a.token_weight) w = a.token_weight[row];
        if (a.seq_coef) coef = a.seq_coef[b];
        scale = a.row_scale[b];
        if (a.ent_weight) h = a.ent_weight[row];
    }
    T* out = static_cast<T*>(a.dlogits) + b * a.out_seq_stride + to * a.out_row_stride;
    typedef typename std::conditional<RAGGED, u32x4_u, u32x4>::type OutVec;
    // RAGGED: `head` elements before the logits row's first 16-byte boundary, `nv` whole vectors from there, then the
    // last elements; lane tid < head + tail owns edge element number `edge` of the row
    int head = 0, edge = -1;
    if constexpr (RAGGED) {
        const T* row0 = static_cast<const T*>(a.logits) + b * a.seq_stride + (inside ? t : 0) * a.row_stride;
        head = int(min(a.vocab, int64_t(((16 - (reinterpret_cast<uintptr_t>(row0) & 15)) & 15) / sizeof(T))));
        nv = int((a.vocab - head) / EPV);
        const int tail0 = head + nv * EPV;
        if (tid < head)
            edge = tid;
        else if (tid - head < int(a.vocab) - tail0)
            edge = tail0 + (tid - head);
    }
    OutVec* op = reinterpret_cast<OutVec*>(out + head);
    if (m == 0.f) {  // no gradient reaches this row: zero-fill
        const u32x4 z = {0u, 0u, 0u, 0u};
        for (int v = tid; v < nv; v += kFThreads) __builtin_nontemporal_store(z, op + v);
        if (RAGGED && edge >= 0) E::store1(out + edge, 0.f);
    }
    if (m == 0.f && !(inside && a.all_rows)) {  // and nothing is read
        if (inside && tid == 0) {
            a.out_logp[row] = 0.f;
            a.out_entropy[row] = 0.f;
            a.out_lse[row] = 0.f;
        }
        return;
    }
    const T* base = static_cast<const T*>(a.logits) + b * a.seq_stride + t * a.row_stride;
    const u32x4* vp = reinterpret_cast<const u32x4*>(base + head);
    const float inv_t = 1.f / a.temperature, c = kLog2e * inv_t;
    // sums of 2^(x c - r0) and of the same times x
    float r0 = 0.f, s = 0.f, u = 0.f;
    [[maybe_unused]] bool have_r0 = false;
    if constexpr (RAGGED) {
        if (edge >= 0) {
            const float x = E::load1(base + edge);
            r0 = ceilf(x * c);
            have_r0 = true;
            s = fast_exp2(fmaf(x, c, -r0));
            u = s * x;
        }
    }
    constexpr int kOnChip = (NVEC + NLDS) * kFThreads;  // vectors of the row the workgroup holds
    if constexpr (EXTRA) {
        for (int v0 = kOnChip; v0 < nv; v0 += 4 * kFThreads) {
            u32x4 e4[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) e4[k] = vp[min(v0 + k * kFThreads + tid, nv - 1)];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                if (v0 + k * kFThreads + tid < nv) {
                    float x[EPV];
                    E::unpack(e4[k], x);
                    if (!have_r0) {
                        float mx = x[0];
#pragma unroll
                        for (int i = 1; i < EPV; ++i) mx = fmaxf(mx, x[i]);
                        r0 = ceilf(mx * c);
                        have_r0 = true;
                    }
#pragma unroll
                    for (int i = 0; i < EPV; ++i) {
                        const float e = fast_exp2(fmaf(x[i], c, -r0));
                        s += e;
                        u = fmaf(e, x[i], u);
                    }
                }
            }
        }
    }
    if constexpr (NLDS > 0) {
        const uint32_t lds0 = uint32_t(reinterpret_cast<uintptr_t>(overflow)) +
                              uint32_t(__builtin_amdgcn_readfirstlane(wave)) * (kWave * 16);
#pragma unroll
        for (int jl = 0; jl < NLDS; ++jl) {
            const int v0 = (NVEC + jl) * kFThreads;
            if (v0 < nv) {  // (uniform over the workgroup; lanes beyond the row's end re-read its last vector)
                const int tj = min(tid, nv - 1 - v0);
                lds_transfer(vp + v0 + tj, lds0 + uint32_t(jl) * (kFThreads * 16));
            }
        }
    }
    u32x4 q[NVEC];
#pragma unroll
    for (int j = 0; j < NVEC; ++j) {
        // the address is (uniform base of vector j, in scalar registers) + the lane's index: one vector register
        // serves all NVEC loads and stores instead of one offset register each.  (Pointers that pass through the
        // empty asm must say that they point to global memory, or the accesses become flat ones, whose waits are
        // all-or-nothing.)
        GlobalVecIn* vj = (GlobalVecIn*)vp + j * kFThreads;
        asm volatile("" : "+s"(vj));
        int tj = tid;
        if (j >= kTail) tj = min(tid, nv - 1 - j * kFThreads);  // (a lane beyond the row's end re-reads the last vector and ignores it)
        q[j] = vj[tj];  // (plain loads: non-temporal ones measure the same to 1 % either way)
    }
    const bool idx_ok = idx >= 0 && idx < a.vocab;
    T x_t_raw = base[idx_ok ? idx : 0];  // requested right behind the row; converted only when the sums are done

    // the sums, vector by vector as the loads retire
#pragma unroll
    for (int j = 0; j < NVEC; ++j) {
        asm volatile("" : "+v"(q[j]));  // (pins the order: vector j is waited for and consumed before vector j + 1)
        if (j < kTail || j * kFThreads + tid < nv) {
            float x[EPV];
            E::unpack(q[j], x);
            if (j == 0 && !((EXTRA || RAGGED) && have_r0)) {
                float mx = x[0];
#pragma unroll
                for (int i = 1; i < EPV; ++i) mx = fmaxf(mx, x[i]);
                r0 = ceilf(mx * c);
            }
#pragma unroll
            for (int i = 0; i < EPV; ++i) {
                const float e = fast_exp2(fmaf(x[i], c, -r0));
                s += e;
                u = fmaf(e, x[i], u);
            }
        }
    }
    const u32x4* lds_q = reinterpret_cast<const u32x4*>(overflow) + tid;  // + jl * kFThreads
    if constexpr (NLDS > 0) {
        // the transfers were issued before every register load and loads return in order: they have landed
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll 1  // (one vector at a time: the registers are full of the row)
        for (int jl = 0; jl < NLDS; ++jl) {
            if ((NVEC + jl) * kFThreads + tid < nv) {
                float x[EPV];
                E::unpack(lds_q[jl * kFThreads], x);
#pragma unroll
                for (int i = 0; i < EPV; ++i) {
                    const float e = fast_exp2(fmaf(x[i], c, -r0));
                    s += e;
                    u = fmaf(e, x[i], u);
                }
            }
        }
    }
    // bring the lanes' sums to a common exponent K >= r0 + log2(s) of every lane
    int es = 0;
    (void)frexpf(s, &es);
    const bool has_data = tid < nv || (RAGGED && edge >= 0);
    const float key = has_data ? r0 + float(es) : -INFINITY;
    const bool bad = !(s < INFINITY) || !(fabsf(u) < INFINITY);  // overflow of a term, or inf / NaN in the row
    const float wk = wave_max(key);
    const bool wbad = __any(bad);
    if (lane == 0) {
        red[0][wave] = wk;
        red[3][wave] = wbad ? 1.f : 0.f;
    }
    __syncthreads();
    float K = -INFINITY, any_bad = 0.f;
#pragma unroll
    for (int k = 0; k < kFWaves; ++k) {
        K = fmaxf(K, red[0][k]);
        any_bad += red[3][k];
    }
    float lse2;  // log2 of sum exp(z), z = x / T
    float S = 0.f, U = 0.f;
    if (any_bad == 0.f) {
        const int sh = int(fminf(fmaxf(r0 - K, -300.f), 300.f));
        s = wave_sum(ldexpf(s, sh));
        u = wave_sum(ldexpf(u, sh));
        if (lane == 0) {
            red[1][wave] = s;
            red[2][wave] = u;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < kFWaves; ++k) {
            S += red[1][k];
            U += red[2][k];
        }
        lse2 = K + __builtin_amdgcn_logf(S);
    } else {
        // the exact reduction: the row's maximum first, then the sums relative to it.  Rare, so it re-reads the row
        // from memory instead of competing with the fast path for the registers that hold it.
        float lm = -INFINITY;
        for (int v = tid; v < nv; v += kFThreads) {
            float x[EPV];
            E::unpack(vp[v], x);
#pragma unroll
            for (int i = 0; i < EPV; ++i) lm = fmaxf(lm, x[i]);
        }
        if (RAGGED && edge >= 0) lm = fmaxf(lm, E::load1(base + edge));
        float M = wave_max(lm);
        if (lane == 0) red[4][wave] = M;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < kFWaves; ++k) M = fmaxf(M, red[4][k]);
        const float mc = M * c;
        s = 0.f;
        u = 0.f;
        for (int v = tid; v < nv; v += kFThreads) {
            float x[EPV];
            E::unpack(vp[v], x);
#pragma unroll
            for (int i = 0; i < EPV; ++i) {
                const float e = fast_exp2(fmaf(x[i], c, -mc));
                s += e;
                u = fmaf(e, x[i], u);
            }
        }
        if (RAGGED && edge >= 0) {
            const float x = E::load1(base + edge);
            const float e = fast_exp2(fmaf(x, c, -mc));
            s += e;
            u = fmaf(e, x, u);
        }
        s = wave_sum(s);
        u = wave_sum(u);
        if (lane == 0) {
            red[5][wave] = s;
            red[6][wave] = u;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < kFWaves; ++k) {
            S += red[5][k];
            U += red[6][k];
        }
        lse2 = mc + __builtin_amdgcn_logf(S);
    }
    // (the compiler must not keep the unpacked values of one sweep alive for the next: 8 floats per vector and lane)
#pragma unroll
    for (int j = 0; j < NVEC; ++j) asm volatile("" : "+v"(q[j]));
    asm volatile("" : "+v"(x_t_raw));
    const float x_t = idx_ok ? E::to_float(x_t_raw) : NAN;
    const float lse = lse2 * kLn2;
    const float ent = lse - (U / S) * inv_t;
    const float lp = x_t * inv_t - lse;
    if (tid == 0) {
        a.out_logp[row] = lp;
        a.out_entropy[row] = ent;
        a.out_lse[row] = lse;
        if (!idx_ok && a.error_flag) atomicOr(a.error_flag, TRLK_FLAG_INDEX_OUT_OF_RANGE);
    }
    if (m == 0.f) return;  // (all_rows) the row was read for its outputs only
    // the token's loss terms -> d loss / d logp, already normalised
    const float c_raw = a.old_logp ? expf(lp - old_lp) : 1.f;
    const PolicyTerm p = policy_term(a, c_raw, A, lp, coef);
    float pl, kl, g_lnc, g_lp;
    grpo_token_terms(a, p, c_raw, lp, w, ref_lp, pl, kl, g_lnc, g_lp);
    float g = (g_lp + g_lnc) * m * scale;
    if (!idx_ok) g = 0.f;  // an invalid index leaves a zero row (its log-prob is NaN and the flag is set)
    // dlogits[v] = p_v (a0 + b0 tt_v) (+ g / T at the target), p_v = 2^tt_v, tt_v = x c - lse2 = (z_v - lse) log2(e):
    // -g p_v / T from the log-prob, -h p_v ((z_v - lse) + H) / T from the entropy
    // Without an entropy term (h == 0, uniform over the workgroup) the factor is the constant a0: a logit of -inf
    // (a masked vocabulary entry) then gets the gradient 0 it has in the reference, where b0 * tt would be 0 * -inf,
    // and an entropy that is NaN for such a row (as the reference's is) stays out of the gradient.
    const bool with_h = h != 0.f;
    const float a0 = with_h ? (-g - h * ent) * inv_t : -g * inv_t;
    const float b0 = with_h ? -h * kLn2 * inv_t : 0.f;
#pragma unroll
    for (int j = 0; j < NVEC; ++j) {
        const int v = j * kFThreads + tid;
        if (j < kTail || v < nv) {
            float x[EPV], d[EPV];
            E::unpack(q[j], x);
#pragma unroll
            for (int i = 0; i < EPV; ++i) {
                const float tt = fmaf(x[i], c, -lse2);
                d[i] = fast_exp2(tt) * (with_h ? fmaf(b0, tt, a0) : a0);
            }
            typedef typename std::conditional<RAGGED, GlobalVecOutU, GlobalVecOut>::type GOut;
            GOut* oj = (GOut*)op + j * kFThreads;
            asm volatile("" : "+s"(oj));
            __builtin_nontemporal_store(E::pack(d), oj + tid);  // (streaming stores: 2-3 % faster than plain ones here)
        }
    }
    if constexpr (NLDS > 0) {
#pragma unroll 1
        for (int jl = 0; jl < NLDS; ++jl) {
            const int v = (NVEC + jl) * kFThreads + tid;
            if (v < nv) {
                float x[EPV], d[EPV];
                E::unpack(lds_q[jl * kFThreads], x);
#pragma unroll
                for (int i = 0; i < EPV; ++i) {
                    const float tt = fmaf(x[i], c, -lse2);
                    d[i] = fast_exp2(tt) * (with_h ? fmaf(b0, tt, a0) : a0);
                }
                __builtin_nontemporal_store(E::pack(d), op + v);
            }
        }
    }
    if constexpr (EXTRA) {
        for (int v0 = kOnChip; v0 < nv; v0 += 4 * kFThreads) {
            u32x4 e4[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) e4[k] = vp[min(v0 + k * kFThreads + tid, nv - 1)];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int v = v0 + k * kFThreads + tid;
                if (v < nv) {
                    float x[EPV], d[EPV];
                    E::unpack(e4[k], x);
#pragma unroll
                    for (int i = 0; i < EPV; ++i) {
                        const float tt = fmaf(x[i], c, -lse2);
                        d[i] = fast_exp2(tt) * (with_h ? fmaf(b0, tt, a0) : a0);
                    }
                    __builtin_nontemporal_store(E::pack(d), op + v);
                }
            }
        }
    }
    if constexpr (RAGGED) {
        if (edge >= 0) {
            const float tt = fmaf(E::load1(base + edge), c, -lse2);
            E::store1(out + edge, fast_exp2(tt) * (with_h ? fmaf(b0, tt, a0) : a0));
        }
    }
    // one-hot term: the lane that stored the target's vector (or edge element) rewrites that element (same lane,
    // same address: ordered after its first store)
    int owner = int((idx / EPV) % kFThreads);
    if constexpr (RAGGED) {
        const int64_t tail0 = head + int64_t(nv) * EPV;
        owner = idx < head ? int(idx) : idx >= tail0 ? head + int(idx - tail0) : int(((idx - head) / EPV) % kFThreads);
    }
    if (idx_ok && owner == tid) {
        const float tt = fmaf(x_t, c, -lse2);
        E::store1(out + idx, fast_exp2(tt) * (with_h ? fmaf(b0, tt, a0) : a0) + g * inv_t);
    }
}

// dynamic LDS above 64 KiB has to be allowed per kernel and device once (a process-wide record: the thread that
// launches need not be the one that called trlk_init)
template <typename Kern>
int reserve_overflow_lds(Kern kern, int bytes) {
    struct Done {
        const void* kern;
        int device;
    };
    static std::mutex guard;
    static std::vector<Done> configured;
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) device = 0;
    const void* key = reinterpret_cast<const void*>(kern);
    std::lock_guard<std::mutex> lock(guard);
    for (const Done& c : configured)
        if (c.kern == key && c.device == device) return TRLK_OK;
    const hipError_t e = hipFuncSetAttribute(key, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return fail(int(e), "grpo_fused: cannot reserve %d bytes of LDS: %s", bytes, hipGetErrorString(e));
    configured.push_back(Done{key, device});
    return TRLK_OK;
}

template <int DT, int NLDS, bool EXTRA, bool R>
int reserve_one() {
    return reserve_overflow_lds(grpo_fused_kernel<DT, kWideVec, NLDS, EXTRA, R>, NLDS * kFThreads * 16);
}
template <int DT, bool R>
int reserve_dtype() {
    if (int rc = reserve_one<DT, 3, false, R>()) return rc;
    if (int rc = reserve_one<DT, 6, false, R>()) return rc;
    if (int rc = reserve_one<DT, 9, false, R>()) return rc;
    return reserve_one<DT, kMaxLdsVec, true, R>();
}

template <int DT, int NLDS, bool EXTRA, bool R>
int launch_fused_wide(const FusedArgs& a, unsigned rows, hipStream_t s) {
    constexpr int kBytes = NLDS * kFThreads * 16;
    if (int rc = reserve_overflow_lds(grpo_fused_kernel<DT, kWideVec, NLDS, EXTRA, R>, kBytes)) return rc;
    hipLaunchKernelGGL((grpo_fused_kernel<DT, kWideVec, NLDS, EXTRA, R>), dim3((rows + 7) / 8 * 8), dim3(kFThreads), kBytes, s, a);
    return TRLK_OK;
}

// R: rows that are not whole aligned vectors
template <int DT, bool R>
int launch_fused(const FusedArgs& a, int nvec, unsigned rows, hipStream_t s) {
    if (nvec > kWideVec + kMaxLdsVec) return launch_fused_wide<DT, kMaxLdsVec, true, R>(a, rows, s);
    if (nvec > kMaxVec) {
        switch ((nvec - kWideVec + kLdsStep - 1) / kLdsStep) {
            case 1: return launch_fused_wide<DT, 3, false, R>(a, rows, s);
            case 2: return launch_fused_wide<DT, 6, false, R>(a, rows, s);
            default: return launch_fused_wide<DT, 9, false, R>(a, rows, s);
        }
    }
    switch ((nvec + kVecStep - 1) / kVecStep) {
        case 1: hipLaunchKernelGGL((grpo_fused_kernel<DT, 4, 0, false, R>), dim3((rows + 7) / 8 * 8), dim3(kFThreads), 0, s, a); break;
        case 2: hipLaunchKernelGGL((grpo_fused_kernel<DT, 8, 0, false, R>), dim3((rows + 7) / 8 * 8), dim3(kFThreads), 0, s, a); break;
        case 3: hipLaunchKernelGGL((grpo_fused_kernel<DT, 12, 0, false, R>), dim3((rows + 7) / 8 * 8), dim3(kFThreads), 0, s, a); break;
        case 4: hipLaunchKernelGGL((grpo_fused_kernel<DT, 16, 0, false, R>), dim3((rows + 7) / 8 * 8), dim3(kFThreads), 0, s, a); break;
        default: hipLaunchKernelGGL((grpo_fused_kernel<DT, 20, 0, false, R>), dim3((rows + 7) / 8 * 8), dim3(kFThreads), 0, s, a); break;
    }
    return TRLK_OK;
}

template <int DT>
int launch_fused_any(const FusedArgs& a, int nvec, bool ragged, unsigned rows, hipStream_t s) {
    return ragged ? launch_fused<DT, true>(a, nvec, rows, s) : launch_fused<DT, false>(a, nvec, rows, s);
}

// data *= *scale over 16-byte vectors, unless the scale is exactly 1 (then nothing is read or written, and what the
// launch costs is the dispatch of its workgroups: each takes 64 pieces of 16 KiB so that a 20 GB buffer needs 19 000
// of them, a few microseconds, where one workgroup per 4 KiB costs a whole millisecond).  The buffer is cut into eight
// contiguous regions, one per XCD (the hardware deals consecutive workgroups to the XCDs in turn), and the workgroups
// of a region step through it together, piece by piece, so that what is read and written at one time is one narrow
// window per XCD.
constexpr int kScalePieceVec = 1024;  // vectors per piece (16 KiB): four per lane in flight
constexpr int kScalePieces = 64;      // pieces per workgroup
template <int DT>
__global__ __launch_bounds__(256) void scale_unless_one_kernel(u32x4* data, int64_t n_vec, int n_tail, const float* scale) {
    typedef Elem<DT> E;
    const float sc = *scale;
    if (sc == 1.f) return;
    if (blockIdx.x == 0 && int(threadIdx.x) < n_tail) {  // the elements after the last whole vector
        typename E::type* p = reinterpret_cast<typename E::type*>(data + n_vec) + threadIdx.x;
        E::store1(p, E::load1(p) * sc);
    }
    const int64_t n_pieces = (n_vec + kScalePieceVec - 1) / kScalePieceVec;
    const int64_t per_xcd = (n_pieces + 7) >> 3;
    const int64_t slots = int64_t(gridDim.x) >> 3;  // the host launches a multiple of eight workgroups
    const int64_t first = int64_t(blockIdx.x & 7) * per_xcd;
#pragma unroll 1
    for (int64_t c = blockIdx.x >> 3; c < per_xcd && first + c < n_pieces; c += slots) {
        u32x4 q[4];
        const int64_t v0 = (first + c) * kScalePieceVec + threadIdx.x;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (v0 + j * 256 < n_vec) q[j] = __builtin_nontemporal_load(data + v0 + j * 256);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (v0 + j * 256 >= n_vec) continue;
            float x[E::EPV];
            E::unpack(q[j], x);
#pragma unroll
            for (int i = 0; i < E::EPV; ++i) x[i] *= sc;
            __builtin_nontemporal_store(E::pack(x), data + v0 + j * 256);
        }
    }
}

}  // namespace

// Every build of the single-pass kernel that keeps part of a row in LDS, allowed its LDS on the current device: what a
// caller does through trlk_init before it captures a graph, so that no launch inside the capture has to.
int grpo_fused_reserve_lds() {
    if (int rc = reserve_dtype<TRLK_BF16, false>()) return rc;
    if (int rc = reserve_dtype<TRLK_BF16, true>()) return rc;
    if (int rc = reserve_dtype<TRLK_F16, false>()) return rc;
    if (int rc = reserve_dtype<TRLK_F16, true>()) return rc;
    if (int rc = reserve_dtype<TRLK_F32, false>()) return rc;
    return reserve_dtype<TRLK_F32, true>();
}
}  // namespace trlk

using namespace trlk;

extern "C" int trlk_scale_unless_one(void* d_data, int dtype, int64_t n_elems, const float* d_scale, trlk_stream_t stream) {
    clear_error();
    TRLK_REQUIRE(dtype == TRLK_BF16 || dtype == TRLK_F16 || dtype == TRLK_F32, TRLK_ERR_BAD_DTYPE,
                 "scale_unless_one: bf16, fp16 or fp32 data (dtype code %d)", dtype);
    const int64_t epv = dtype == TRLK_F32 ? 4 : 8;
    TRLK_REQUIRE(n_elems >= 0, TRLK_ERR_BAD_SHAPE, "scale_unless_one: negative element count");
    if (n_elems == 0) return TRLK_OK;
    TRLK_REQUIRE(d_data && d_scale && reinterpret_cast<uintptr_t>(d_data) % 16 == 0, TRLK_ERR_NULL_POINTER,
                 "scale_unless_one: null or misaligned pointer");
    const int64_t n_vec = n_elems / epv;
    const int n_tail = int(n_elems - n_vec * epv);
    const int64_t n_pieces = (n_vec + kScalePieceVec - 1) / kScalePieceVec;
    const int64_t slots = ((n_pieces + 7) / 8 + kScalePieces - 1) / kScalePieces;  // workgroups per region
    TRLK_REQUIRE(slots <= 0x0fffffff, TRLK_ERR_BAD_SHAPE, "scale_unless_one: too many elements");
    const unsigned grid = 8u * unsigned(slots > 0 ? slots : 1);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == TRLK_BF16)
        hipLaunchKernelGGL(scale_unless_one_kernel<TRLK_BF16>, dim3(grid), dim3(256), 0, s, static_cast<u32x4*>(d_data), n_vec, n_tail, d_scale);
    else if (dtype == TRLK_F16)
        hipLaunchKernelGGL(scale_unless_one_kernel<TRLK_F16>, dim3(grid), dim3(256), 0, s, static_cast<u32x4*>(d_data), n_vec, n_tail, d_scale);
    else
        hipLaunchKernelGGL(scale_unless_one_kernel<TRLK_F32>, dim3(grid), dim3(256), 0, s, static_cast<u32x4*>(d_data), n_vec, n_tail, d_scale);
    return launch_status("scale_unless_one");
}

extern "C" int64_t trlk_grpo_fused_max_vocab(int dtype) {
    const int64_t vectors = int64_t(kWideVec + kMaxLdsVec + kMaxExtraVec) * kFThreads;
    return dtype == TRLK_BF16 || dtype == TRLK_F16 ? vectors * 8 : dtype == TRLK_F32 ? vectors * 4 : 0;
}

extern "C" int trlk_grpo_fused_fwd_bwd(const void* d_logits, int dtype, int64_t n_seq, int64_t rows_per_seq, int64_t vocab,
                                       int64_t seq_stride, int64_t row_stride, const int64_t* d_index, float temperature,
                                       const float* d_old_logp, const float* d_ref_logp, const float* d_advantages,
                                       int64_t adv_stride_b, int64_t adv_stride_t, const float* d_mask,
                                       const float* d_token_weight, const float* d_seq_coef, const float* d_row_scale,
                                       const float* d_entropy_weight, int policy_term, float epsilon_low, float epsilon_high, float delta, float beta,
                                       int use_bias_correction_kl, float sapo_temperature_pos, float sapo_temperature_neg,
                                       float* d_out_logp, float* d_out_entropy, float* d_out_lse, void* d_dlogits,
                                       int64_t out_rows_per_seq, int64_t out_row_offset, int64_t out_seq_stride,
                                       int64_t out_row_stride, int compute_masked_rows, int32_t* d_error_flag,
                                       trlk_stream_t stream) {
    clear_error();
    TRLK_REQUIRE(dtype == TRLK_BF16 || dtype == TRLK_F16 || dtype == TRLK_F32, TRLK_ERR_BAD_DTYPE,
                 "grpo_fused: bf16, fp16 or fp32 logits (dtype code %d); use the two-pass path", dtype);
    const int64_t es = int64_t(elem_size(dtype)), epv = 16 / es;
    TRLK_REQUIRE(n_seq >= 0 && rows_per_seq >= 0 && vocab >= 1, TRLK_ERR_BAD_SHAPE, "grpo_fused: bad sizes");
    TRLK_REQUIRE(vocab >= epv && vocab <= trlk_grpo_fused_max_vocab(dtype), TRLK_ERR_UNSUPPORTED,
                 "grpo_fused: vocab must be at least %lld and at most %lld (got %lld); use the two-pass path",
                 (long long)epv, (long long)trlk_grpo_fused_max_vocab(dtype), (long long)vocab);
    TRLK_REQUIRE(out_row_offset >= 0 && out_row_offset + rows_per_seq <= out_rows_per_seq, TRLK_ERR_BAD_SHAPE,
                 "grpo_fused: input rows [%lld, %lld) do not fit the %lld output rows per sequence",
                 (long long)out_row_offset, (long long)(out_row_offset + rows_per_seq), (long long)out_rows_per_seq);
    TRLK_REQUIRE(temperature > 0.f && temperature < INFINITY, TRLK_ERR_BAD_VALUE,
                 "grpo_fused: temperature must be positive and finite (got %g)", (double)temperature);
    TRLK_REQUIRE(policy_term >= TRLK_TERM_CLIP && policy_term <= TRLK_TERM_WEIGHTED_LOGP, TRLK_ERR_BAD_VALUE,
                 "grpo_fused: unknown policy term %d", policy_term);
    const int64_t orows = n_seq * out_rows_per_seq;
    if (orows == 0) return TRLK_OK;
    TRLK_REQUIRE(orows < (int64_t(1) << 31) - 8, TRLK_ERR_BAD_SHAPE, "grpo_fused: too many rows (%lld)", (long long)orows);
    TRLK_REQUIRE(d_dlogits != nullptr, TRLK_ERR_NULL_POINTER, "grpo_fused: dlogits pointer is null");
    if (n_seq * rows_per_seq > 0) {
        TRLK_REQUIRE(d_logits && d_index && d_advantages && d_mask && d_row_scale && d_out_logp && d_out_entropy && d_out_lse,
                     TRLK_ERR_NULL_POINTER, "grpo_fused: a required pointer is null");
        TRLK_REQUIRE(beta == 0.f || d_ref_logp != nullptr, TRLK_ERR_NULL_POINTER, "grpo_fused: beta != 0 needs ref_logp");
        TRLK_REQUIRE(policy_term != TRLK_TERM_WEIGHTED_LOGP || d_seq_coef != nullptr, TRLK_ERR_NULL_POINTER,
                     "grpo_fused: the weighted log-prob term needs seq_coef");
        TRLK_REQUIRE(row_stride >= vocab || rows_per_seq <= 1, TRLK_ERR_BAD_STRIDE, "grpo_fused: rows overlap");
    }
    const auto al16 = [es](const void* p, int64_t s0, int64_t s1) {
        return reinterpret_cast<uintptr_t>(p) % 16 == 0 && (s0 * es) % 16 == 0 && (s1 * es) % 16 == 0;
    };
    TRLK_REQUIRE(reinterpret_cast<uintptr_t>(d_logits) % es == 0 && reinterpret_cast<uintptr_t>(d_dlogits) % es == 0,
                 TRLK_ERR_BAD_STRIDE, "grpo_fused: logits and dlogits must be aligned to their element size");
    // rows that are not whole aligned vectors take the builds that peel a row to its first 16-byte boundary
    const bool ragged = vocab % epv != 0 || !al16(d_logits, seq_stride, row_stride) ||
                        !al16(d_dlogits, out_seq_stride, out_row_stride);
    // (a peeled row must still hold one whole vector)
    TRLK_REQUIRE(!ragged || vocab >= 2 * epv, TRLK_ERR_UNSUPPORTED,
                 "grpo_fused: rows that are not whole aligned vectors need at least %lld entries (got %lld); use the two-pass path",
                 (long long)(2 * epv), (long long)vocab);
    FusedArgs a{};
    a.logits = d_logits;
    a.rows_per_seq = rows_per_seq;
    a.vocab = vocab;
    a.seq_stride = seq_stride;
    a.row_stride = row_stride;
    a.index = d_index;
    a.temperature = temperature;
    a.old_logp = d_old_logp;
    a.ref_logp = d_ref_logp;
    a.adv = d_advantages;
    a.mask = d_mask;
    a.token_weight = d_token_weight;
    a.row_scale = d_row_scale;
    a.ent_weight = d_entropy_weight;
    a.seq_coef = d_seq_coef;
    a.adv_stride_b = adv_stride_b;
    a.adv_stride_t = adv_stride_t;
    a.policy_term = policy_term;
    a.eps_low = epsilon_low;
    a.eps_high = epsilon_high;
    a.delta = delta;
    a.beta = beta;
    a.bias_kl = use_bias_correction_kl;
    a.sapo_tau_pos = sapo_temperature_pos;
    a.sapo_tau_neg = sapo_temperature_neg;
    a.out_logp = d_out_logp;
    a.out_entropy = d_out_entropy;
    a.out_lse = d_out_lse;
    a.dlogits = d_dlogits;
    a.out_rows_per_seq = out_rows_per_seq;
    a.out_row_offset = out_row_offset;
    a.out_seq_stride = out_seq_stride;
    a.out_row_stride = out_row_stride;
    a.error_flag = d_error_flag;
    a.all_rows = compute_masked_rows != 0;
    a.total_rows = orows;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int nvec = int((vocab / epv + kFThreads - 1) / kFThreads);  // 16-byte vectors of the row per lane
    if (int rc = dtype == TRLK_BF16  ? launch_fused_any<TRLK_BF16>(a, nvec, ragged, unsigned(orows), s)
                 : dtype == TRLK_F16 ? launch_fused_any<TRLK_F16>(a, nvec, ragged, unsigned(orows), s)
                                     : launch_fused_any<TRLK_F32>(a, nvec, ragged, unsigned(orows), s))
        return rc;
    return launch_status("grpo_fused");
}
