// K1 / K3: streaming log-prob + entropy forward and its recompute backward.
//
// One workgroup owns one row (token position).  The row is streamed once with 16-byte
// non-temporal loads, `UNR` loads in flight per lane; every lane keeps an online
// (reference exponent r, sum 2^(x*c-r), sum 2^(x*c-r)*x) triple in fp32 and the triples are merged
// across the workgroup through wave shuffles and LDS.  The temperature is folded into the
// exponent multiplier (c = log2(e)/T), so no scaled copy of the row ever exists.
// The backward re-streams the row and the saved lse and writes dlogits in the same pass.
#include "common.hpp"

namespace trlk {
namespace {

// Tuning knobs (overridable with -D for experiments; the defaults are the measured best on the
// [65536, 151936] bf16 workload).  Forward: 4 non-temporal 16-byte loads in flight per lane.
// Backward: 8 KiB chunks (2 loads per lane), plain loads, non-temporal stores.
#ifndef TRLK_THREADS
#define TRLK_THREADS 256
#endif
#ifndef TRLK_FWD_UNROLL
#define TRLK_FWD_UNROLL 4
#endif
#ifndef TRLK_BWD_UNROLL
#define TRLK_BWD_UNROLL 2
#endif
#ifndef TRLK_FWD_NT_LOAD
#define TRLK_FWD_NT_LOAD 1
#endif
#ifndef TRLK_BWD_NT_LOAD
#define TRLK_BWD_NT_LOAD 1  // (with every XCD on its own region of the chunks: 2-3 % ahead of plain loads; no difference before)
#endif
#ifndef TRLK_NT_STORE
#define TRLK_NT_STORE 1
#endif
constexpr int kThreads = TRLK_THREADS;
constexpr int kUnroll = TRLK_FWD_UNROLL;
static_assert(kUnroll >= 2, "the row tail of the forward holds up to kUnroll - 1 vectors per lane");
constexpr int kBwdUnroll = TRLK_BWD_UNROLL;

// A 16-byte vector at any element alignment: rows whose length is no multiple of the vector width start at 2- or
// 4-byte aligned addresses.  The hardware takes such accesses as they are (one instruction; a wave's kilobyte then
// touches nine cache lines instead of eight).
typedef u32x4 u32x4_u __attribute__((aligned(2)));
template <bool ALIGNED>
struct VecOf {
    typedef u32x4 type;
};
template <>
struct VecOf<false> {
    typedef u32x4_u type;
};

template <bool NT, typename V>
__device__ __forceinline__ u32x4 stream_load(const V* p) {
    if constexpr (NT)
        return __builtin_nontemporal_load(p);
    else
        return *p;
}
template <typename V>
__device__ __forceinline__ void stream_store(u32x4 v, V* p) {
#if TRLK_NT_STORE
    __builtin_nontemporal_store(v, p);
#else
    *p = v;
#endif
}
constexpr bool kFwdNt = TRLK_FWD_NT_LOAD != 0;
constexpr bool kBwdNt = TRLK_BWD_NT_LOAD != 0;
constexpr int kMaxIndex = 64;  // most indices per row the backward accepts

struct FwdArgs {
    const void* logits;
    int64_t rows_per_seq, vocab, seq_stride, row_stride;
    const int64_t* index;
    int32_t n_index;
    float temperature;
    const uint8_t* row_mask;
    float* out_logp;
    float* out_entropy;
    float* out_lse;
    float* out_stats;  // [rows, 4] or null: mean logit, log sum_v p_v^2, first index is the arg-max, 0
    int32_t* error_flag;
};

// Per-lane online log-sum-exp state in base 2.  The reference point `r` is an INTEGER (held in a
// float): ceil(max * c) of the values seen so far.  exp2(x*c - r) then has no rounding in the
// reference itself (the fma rounds once, relative to the small difference near the maximum), and
// moving to a larger reference is an exact power-of-two rescale.
struct OnlineLse {
    float r = -INFINITY;  // integer reference exponent (-inf until a finite value was seen)
    float rr = 0.f;       // r, with 0 standing in while r is still -inf
    float s = 0.f;        // sum exp2(x*c - r)
    float u = 0.f;        // sum exp2(x*c - r) * x
    __device__ __forceinline__ void raise(float bm, float c) {
        const float need = ceilf(bm * c);
        if (need > r) {
            const float sc = fast_exp2(r - need);  // r = -inf gives 0, and s = u = 0 then
            s *= sc;
            u *= sc;
            r = need;
            rr = need;
        }
    }
    __device__ __forceinline__ void add(float x, float c) {
        const float e = fast_exp2(fmaf(x, c, -rr));
        s += e;
        u = fmaf(e, x, u);
    }
};

// Extra per-lane row statistics of the STATS variant (what the DPO metrics and the WPO weights
// need on top of log-prob and entropy, so that no further pass over the logits is necessary):
// sum of exp2(x*c - r)^2 (same reference as OnlineLse), sum of x, and the lane's running maximum
// with the FIRST position that holds it (a lane visits its positions in increasing order and only
// a strictly larger value moves the position, so ties keep the earliest one, as torch.argmax does).
struct RowStats {
    float s2 = 0.f, sx = 0.f;
    float vmax = -INFINITY;
    float vpos = 3.0e38f;  // position as a float: exact below 2^24, which the host guarantees
};

// sum of the two 16-bit floats packed in w, added to acc (one dot-product instruction against (1, 1))
template <int DT>
__device__ __forceinline__ float add_pair(uint32_t w, float acc) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
    if constexpr (DT == TRLK_BF16)
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w), __builtin_bit_cast(bf16x2_t, 0x3F803F80u),
                                               acc, false);
    else
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, w), __builtin_bit_cast(f16x2_t, 0x3C003C00u), acc, false);
}

template <int N>
__device__ __forceinline__ float max_of(const float* x) {
    float a = x[0];
#pragma unroll
    for (int i = 1; i < N; ++i) a = fmaxf(a, x[i]);
    return a;
}

// VEC: rows are 16-byte aligned and vocab is a multiple of the vector width.  Otherwise a row is read in aligned
// vectors from its first 16-byte boundary on, and the few elements before that and after the last whole vector one by one.
// STATS: 1 or 2 also produce the row statistics of `out_stats`; only 2 accumulates the sum of squared probabilities
// (one more multiply-add per logit in a loop that is bound by its arithmetic: 5.14 against 4.95 ms on 33.6 GB of bf16
// logits), 1 reports 0 in its place.
// TH lanes per row, UN 16-byte loads in flight per lane.
template <int DT, bool VEC, int STATS, int TH = kThreads, int UN = kUnroll>
__global__ __launch_bounds__(TH) void logp_entropy_fwd_kernel(FwdArgs a) {
    static_assert(UN >= 2, "the row tail holds up to UN - 1 vectors per lane");
    typedef Elem<DT> E;
    typedef typename E::type T;
    constexpr int NW = TH / kWave;
    __shared__ float red[STATS ? 7 : 3][NW];
    __shared__ float bcast[2];

    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    if (a.row_mask != nullptr && a.row_mask[row] == 0) {
        for (int k = tid; k < a.n_index; k += TH) a.out_logp[row * a.n_index + k] = 0.f;
        if (tid == 0) {
            if (a.out_entropy) a.out_entropy[row] = 0.f;
            if (a.out_lse) a.out_lse[row] = 0.f;
        }
        if (STATS && tid < 4) a.out_stats[row * 4 + tid] = 0.f;
        return;
    }
    const int64_t b = row / a.rows_per_seq;
    const int64_t t = row - b * a.rows_per_seq;
    const T* base = static_cast<const T*>(a.logits) + b * a.seq_stride + t * a.row_stride;
    const float c = kLog2e / a.temperature;
    const int64_t V = a.vocab;

    OnlineLse acc;
    RowStats st;
    // one element with its position e (stats only)
    auto stat_elem = [&](float x, int64_t e) {
        st.sx += x;
        if (x > st.vmax) {
            st.vmax = x;
            st.vpos = float(e);
        }
    };
    // N elements starting at position e0 whose maximum is bm (q: their packed form, 16-bit types only).  The
    // running maximum moves a few times per row only, so the position search sits in a rarely taken branch.
    // (the sum is taken from the packed form first, so that it need not stay in registers beside the unpacked one)
    auto stat_sum = [&](u32x4 q) {
        if constexpr (DT == TRLK_F32) {
#pragma unroll
            for (int w = 0; w < 4; ++w) st.sx += __uint_as_float(q[w]);
        } else {
#pragma unroll
            for (int w = 0; w < 4; ++w) st.sx = add_pair<DT>(q[w], st.sx);
        }
    };
    auto stat_vec = [&](const float* x, int64_t e0, int n, float bm) {
        if (bm > st.vmax) {
            st.vmax = bm;
            int first = n - 1;
            for (int i = n - 2; i >= 0; --i) first = x[i] == bm ? i : first;
            st.vpos = float(e0 + first);
        }
    };
    auto raise = [&](float bm) {
        if constexpr (STATS == 2) {
            const float need = ceilf(bm * c);
            if (need > acc.r) {
                const float sc = fast_exp2(acc.r - need);
                st.s2 *= sc * sc;
            }
        }
        acc.raise(bm, c);
    };
    auto add = [&](float x) {
        if constexpr (STATS == 2) {
            const float e = fast_exp2(fmaf(x, c, -acc.rr));
            acc.s += e;
            acc.u = fmaf(e, x, acc.u);
            st.s2 = fmaf(e, e, st.s2);
        } else {
            acc.add(x, c);
        }
    };
    {
        constexpr int EPV = E::EPV;
        // Rows that are not whole aligned vectors (not VEC): the `head` elements before the row's first 16-byte
        // boundary go one by one (first: a lane's positions must come in increasing order), then aligned vectors,
        // then what is left after the last whole one.
        const int head = VEC ? 0 : int(min(V, int64_t(((16 - (reinterpret_cast<uintptr_t>(base) & 15)) & 15) / sizeof(T))));
        if constexpr (!VEC) {
            if (tid < head) {
                const float x = E::load1(base + tid);
                raise(x);
                add(x);
                if constexpr (STATS) stat_elem(x, tid);
            }
        }
        const u32x4* vp = reinterpret_cast<const u32x4*>(base + head);
        const int nvec = int((V - head) / EPV);
        int v = tid;
        for (; v + (UN - 1) * TH < nvec; v += UN * TH) {
            u32x4 q[UN];
#pragma unroll
            for (int j = 0; j < UN; ++j) q[j] = stream_load<kFwdNt>(vp + v + j * TH);
            if constexpr (STATS) {
#pragma unroll
                for (int j = 0; j < UN; ++j) stat_sum(q[j]);
            }
            float x[UN * EPV];
#pragma unroll
            for (int j = 0; j < UN; ++j) E::unpack(q[j], x + j * EPV);
            const float bm = max_of<UN * EPV>(x);  // one maximum over the whole group
            raise(bm);
#pragma unroll
            for (int i = 0; i < UN * EPV; ++i) add(x[i]);
            if constexpr (STATS) {
                // the lane's running maximum moves a few times per row: only then is the position looked for, over
                // the group's vectors in the order of their positions (the j-th lies before the (j+1)-th)
                if (bm > st.vmax) {
                    st.vmax = bm;
                    int first = UN * EPV - 1;
                    for (int i = UN * EPV - 2; i >= 0; --i) first = x[i] == bm ? i : first;
                    st.vpos = float(head + int64_t(v + (first / EPV) * TH) * EPV + first % EPV);
                }
            }
        }
        // the row's tail: fewer than UN vectors are left for this lane; their loads go out together
        // (one after the other they would cost a memory round trip each, at the end of every row)
        {
            u32x4 q[UN - 1];
#pragma unroll
            for (int j = 0; j < UN - 1; ++j)
                if (v + j * TH < nvec) q[j] = stream_load<kFwdNt>(vp + v + j * TH);
#pragma unroll
            for (int j = 0; j < UN - 1; ++j) {
                if (v + j * TH < nvec) {
                    if constexpr (STATS) stat_sum(q[j]);
                    float x[EPV];
                    E::unpack(q[j], x);
                    const float bm = max_of<EPV>(x);
                    raise(bm);
#pragma unroll
                    for (int i = 0; i < EPV; ++i) add(x[i]);
                    if constexpr (STATS) stat_vec(x, head + int64_t(v + j * TH) * EPV, EPV, bm);
                }
            }
        }
        if constexpr (!VEC) {  // what is left of the row after its whole vectors (these positions come last for a lane)
            for (int64_t e = head + int64_t(nvec) * EPV + tid; e < V; e += TH) {
                const float x = E::load1(base + e);
                raise(x);
                add(x);
                if constexpr (STATS) stat_elem(x, e);
            }
        }
    }

    // ---- merge the per-lane triples: common reference first (exact rescale), then two sums -----
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    float wr = wave_max(acc.r);
    if (lane == 0) red[0][wave] = wr;
    __syncthreads();
    float R = red[0][0];
#pragma unroll
    for (int w = 1; w < NW; ++w) R = fmaxf(R, red[0][w]);
    // lanes that saw nothing finite have r = -inf and s = 0; a zero factor keeps them out
    const float sc = (acc.r == -INFINITY) ? 0.f : fast_exp2(acc.r - R);
    float s = wave_sum(acc.s * sc);
    float u = wave_sum(acc.u * sc);
    if (lane == 0) {
        red[1][wave] = s;
        red[2][wave] = u;
    }
    if constexpr (STATS) {
        const float s2 = STATS == 2 ? wave_sum(st.s2 * sc * sc) : 0.f;
        const float sx = wave_sum(st.sx);
        // the row maximum and the smallest position among the lanes that hold it
        const float wmax = wave_max(st.vmax);
        const float wpos = wave_min(st.vmax == wmax ? st.vpos : 3.0e38f);
        if (lane == 0) {
            red[3][wave] = s2;
            red[4][wave] = sx;
            red[5][wave] = wmax;
            red[6][wave] = wpos;
        }
    }
    __syncthreads();
    if (tid == 0) {
        float S = 0.f, U = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            S += red[1][w];
            U += red[2][w];
        }
        if constexpr (STATS) {
            float S2 = 0.f, SX = 0.f, vmax = -INFINITY, vpos = 3.0e38f;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                S2 += red[3][w];
                SX += red[4][w];
                if (red[5][w] > vmax || (red[5][w] == vmax && red[6][w] < vpos)) {
                    vmax = red[5][w];
                    vpos = red[6][w];
                }
            }
            const int64_t tpos = a.n_index > 0 ? a.index[row * a.n_index] : -1;
            float* o = a.out_stats + row * 4;
            o[0] = SX / float(V);
            o[1] = STATS == 2 ? logf(S2) - 2.f * logf(S) : 0.f;  // log sum_v softmax(z)_v^2: the common reference cancels
            o[2] = (tpos >= 0 && tpos < V && float(tpos) == vpos) ? 1.f : 0.f;
            o[3] = 0.f;
        }
        // lse = R*ln2 + ln S with ln2 split in two so that the product carries no rounding of ln2
        constexpr float kLn2Hi = 0.693145751953125f, kLn2Lo = 1.42860677e-06f;
        const float lse = fmaf(R, kLn2Hi, fmaf(R, kLn2Lo, logf(S)));
        const float ent = lse - (U / S) / a.temperature;
        bcast[0] = lse;
        if (a.out_entropy) a.out_entropy[row] = ent;
        if (a.out_lse) a.out_lse[row] = lse;
    }
    __syncthreads();
    const float lse = bcast[0];
    for (int k = tid; k < a.n_index; k += TH) {
        const int64_t idx = a.index[row * a.n_index + k];
        float r;
        if (idx < 0 || idx >= V) {
            r = NAN;
            if (a.error_flag) atomicOr(a.error_flag, TRLK_FLAG_INDEX_OUT_OF_RANGE);
        } else {
            r = E::load1(base + idx) / a.temperature - lse;
        }
        a.out_logp[row * a.n_index + k] = r;
    }
}

struct BwdArgs {
    const void* logits;
    int64_t rows_per_seq, vocab, seq_stride, row_stride;
    const int64_t* index;
    int32_t n_index;
    float temperature;
    const float* lse;
    const float* entropy;
    const float* g_logp;
    const float* g_entropy;
    void* dlogits;
    int64_t out_rows_per_seq, out_row_offset, out_seq_stride, out_row_stride;
    int64_t total_chunks;  // rows x chunks per row
};

// The backward has no reduction, so a row is cut into chunks of kChunkElems elements and one
// workgroup handles one chunk of one row; consecutive workgroups then touch consecutive addresses
// (row-major), which keeps the read and write streams of the whole grid inside a narrow,
// DRAM-page-friendly window instead of thousands of rows apart.
constexpr int kChunkBytes = kThreads * kBwdUnroll * 16;

template <int DT>
constexpr int chunk_elems() {
    return kChunkBytes / int(sizeof(typename Elem<DT>::type));
}

// HAS_H: an entropy gradient is present.
template <int DT, bool VEC, bool HAS_H>
__global__ __launch_bounds__(kThreads) void logp_entropy_bwd_kernel(BwdArgs a, int chunks_per_row) {
    typedef Elem<DT> E;
    typedef typename E::type T;
    constexpr int CE = chunk_elems<DT>();

    const int tid = threadIdx.x;
    // The hardware deals consecutive workgroups to the eight XCDs in turn.  Each XCD walks one contiguous eighth of the
    // chunks (address-linear inside it) instead of every eighth chunk of the whole buffer: eight narrow write windows,
    // one per XCD.  Measured on bf16 [64, 1024, 151936]: zero-filled rows 3.39 -> 2.97 ms, the benchmark's prefix mask
    // 5.20 -> 4.95 ms, every row active 6.3 -> 6.5 ms; 16, 32 or 64 such regions are slower than either.
    const int64_t per_xcd = int64_t(gridDim.x) >> 3;  // (the grid is a multiple of 8)
    const int64_t linear = int64_t(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (linear >= a.total_chunks) return;
    const int64_t orow = linear / chunks_per_row;
    const int chunk = int(linear - orow * chunks_per_row);
    const int64_t b = orow / a.out_rows_per_seq;
    const int64_t to = orow - b * a.out_rows_per_seq;
    const int64_t t = to - a.out_row_offset;
    T* out = static_cast<T*>(a.dlogits) + b * a.out_seq_stride + to * a.out_row_stride;
    // Rows that are not whole aligned vectors (not VEC) are walked from the first 16-byte boundary of the OUTPUT row:
    // the `head` elements before it and what is left after the last whole vector go one by one, the vectors between
    // through accesses that need no alignment (when the logits row sits like the gradient row -- two contiguous
    // tensors of one shape -- both sides are in fact aligned).  The chunks count from that boundary.
    const int head = VEC ? 0 : int(min(a.vocab, int64_t(((16 - (reinterpret_cast<uintptr_t>(out) & 15)) & 15) / sizeof(T))));
    const int body = int(a.vocab) - head;
    const int e0 = chunk * CE;                                   // first element of this chunk, counted from `head`
    const int e1 = max(e0, body < e0 + CE ? body : e0 + CE);     // (an empty range in a last chunk that the head made superfluous)
    out += head;

    // Everything below up to the streaming loop is uniform over the workgroup (scalar loads).
    bool live = t >= 0 && t < a.rows_per_seq;
    const int64_t row = b * a.rows_per_seq + (live ? t : 0);
    const int K = a.n_index;
    const float inv_t = 1.f / a.temperature;
    float gsum = 0.f;
    bool any = false;
    if (live) {
        for (int k = 0; k < K; ++k) {
            const float g = a.g_logp[row * K + k];
            gsum += g;
            any |= (g != 0.f);
        }
    }
    const float h = (HAS_H && live) ? a.g_entropy[row] : 0.f;
    live = live && (any || h != 0.f);
    typedef typename VecOf<VEC>::type Vec;  // (not VEC: whole vectors through unaligned accesses, the row's last elements one by one)
    const int v_end = e1 / E::EPV;          // whole vectors of the row end here (e1 is the row's end in its last chunk)
    if (!live) {  // outside the kept window, or all upstream gradients are zero: zero-fill
        Vec* op = reinterpret_cast<Vec*>(out);
        const u32x4 z = {0u, 0u, 0u, 0u};
        for (int v = e0 / E::EPV + tid; v < v_end; v += kThreads) stream_store(z, op + v);
        if constexpr (!VEC) {
            for (int e = v_end * E::EPV + tid; e < e1; e += kThreads) E::store1(out + e, 0.f);
            if (chunk == 0 && tid < head) E::store1(out - head + tid, 0.f);
        }
        return;
    }
    const T* base = static_cast<const T*>(a.logits) + b * a.seq_stride + t * a.row_stride + head;
    const float c = kLog2e * inv_t;
    const float lsec = a.lse[row] * kLog2e;
    // dz_v = p_v * (a0 + b0 * tt),  tt = x*c - lse*log2e = (z - lse) * log2e
    // (a row without an entropy gradient of its own keeps the constant factor: its entropy may be NaN, as the
    // reference's is for a row with -inf logits, and b0 * tt would be 0 * -inf at such a logit)
    const bool with_h = HAS_H && h != 0.f;
    const float a0 = with_h ? (-gsum - h * a.entropy[row]) * inv_t : -gsum * inv_t;
    const float b0 = with_h ? -h * kLn2 * inv_t : 0.f;
    auto grad_of = [&](float x) {
        const float tt = fmaf(x, c, -lsec);
        const float p = fast_exp2(tt);
        return with_h ? p * fmaf(b0, tt, a0) : p * a0;
    };

    {
        constexpr int EPV = E::EPV;
        const Vec* vp = reinterpret_cast<const Vec*>(base);
        Vec* op = reinterpret_cast<Vec*>(out);
        const int v0 = e0 / EPV + tid;
        auto one_vector = [&](u32x4 q, int v) {
            float x[EPV], d[EPV];
            E::unpack(q, x);
#pragma unroll
            for (int i = 0; i < EPV; ++i) d[i] = grad_of(x[i]);
            stream_store(E::pack(d), op + v);
        };
        if (v0 + (kBwdUnroll - 1) * kThreads < v_end) {  // full chunk: all loads first
            u32x4 q[kBwdUnroll];
#pragma unroll
            for (int j = 0; j < kBwdUnroll; ++j) q[j] = stream_load<kBwdNt>(vp + v0 + j * kThreads);
#pragma unroll
            for (int j = 0; j < kBwdUnroll; ++j) one_vector(q[j], v0 + j * kThreads);
        } else {
            for (int v = v0; v < v_end; v += kThreads) one_vector(stream_load<kBwdNt>(vp + v), v);
        }
        if constexpr (!VEC) {
            for (int e = v_end * EPV + tid; e < e1; e += kThreads) E::store1(out + e, grad_of(E::load1(base + e)));
            if (chunk == 0 && tid < head) E::store1(out - head + tid, grad_of(E::load1(base - head + tid)));
        }
    }
    // One-hot terms.  The streaming part above wrote only the softmax term; the lane that stored
    // the element at index[k] now rewrites it with the gathered gradients added (a later store of
    // the same lane to the same address is ordered after the first).  Entries of one row that
    // share an index are summed in k order by the first of them.
    for (int k = 0; k < K; ++k) {
        const int64_t idx = a.index[row * K + k] - head;  // counted from `head` like the chunks
        // this chunk's elements, or (chunk 0) the head; also drops indices outside [0, vocab)
        const bool in_head = !VEC && chunk == 0 && idx < 0 && idx >= -int64_t(head);
        if (!in_head && (idx < e0 || idx >= e1)) continue;
        // (whole vectors: lane (vector number in the chunk) mod kThreads; the elements before and after them: one lane each)
        const int owner = in_head ? int(idx + head)
                                  : idx < int64_t(v_end) * E::EPV ? int((idx - e0) / E::EPV) % kThreads
                                                                  : int(idx - int64_t(v_end) * E::EPV);
        if (owner != tid) continue;
        float add = 0.f;
        bool first = true;
        for (int j = 0; j < K; ++j) {
            if (a.index[row * K + j] - head != idx) continue;
            if (j < k) first = false;
            add += a.g_logp[row * K + j] * inv_t;
        }
        if (!first) continue;
        E::store1(out + idx, grad_of(E::load1(base + idx)) + add);
    }
}

bool aligned16(const void* p, size_t es, std::initializer_list<int64_t> strides) {
    if (reinterpret_cast<uintptr_t>(p) % 16 != 0) return false;
    for (int64_t s : strides)
        if ((s * int64_t(es)) % 16 != 0) return false;
    return true;
}

int check_view(const char* what, const void* p, int dtype, int64_t n_seq, int64_t rows_per_seq, int64_t vocab,
               int64_t seq_stride, int64_t row_stride) {
    TRLK_REQUIRE(dtype == TRLK_F32 || dtype == TRLK_BF16 || dtype == TRLK_F16, TRLK_ERR_BAD_DTYPE,
                 "%s: unsupported dtype code %d", what, dtype);
    TRLK_REQUIRE(n_seq >= 0 && rows_per_seq >= 0, TRLK_ERR_BAD_SHAPE, "%s: negative row count", what);
    TRLK_REQUIRE(vocab >= 1, TRLK_ERR_BAD_SHAPE, "%s: vocab must be >= 1 (got %lld)", what, (long long)vocab);
    TRLK_REQUIRE(vocab < (int64_t(1) << 31) - 16 * kThreads * kUnroll, TRLK_ERR_BAD_SHAPE,
                 "%s: vocab %lld too large", what, (long long)vocab);
    TRLK_REQUIRE(n_seq * rows_per_seq < (int64_t(1) << 31), TRLK_ERR_BAD_SHAPE, "%s: too many rows (%lld)", what,
                 (long long)(n_seq * rows_per_seq));
    if (n_seq * rows_per_seq > 0) {
        TRLK_REQUIRE(p != nullptr, TRLK_ERR_NULL_POINTER, "%s: null data pointer", what);
        TRLK_REQUIRE(row_stride >= vocab || rows_per_seq <= 1, TRLK_ERR_BAD_STRIDE,
                     "%s: row_stride %lld < vocab %lld (rows overlap)", what, (long long)row_stride, (long long)vocab);
        TRLK_REQUIRE(seq_stride >= 0 && row_stride >= 0, TRLK_ERR_BAD_STRIDE, "%s: negative stride", what);
    }
    return TRLK_OK;
}

}  // namespace
}  // namespace trlk

using namespace trlk;

extern "C" int trlk_logp_entropy_fwd(const void* d_logits, int dtype, int64_t n_seq, int64_t rows_per_seq,
                                     int64_t vocab, int64_t seq_stride, int64_t row_stride, const int64_t* d_index,
                                     int32_t n_index, float temperature, const uint8_t* d_row_mask,
                                     float* d_out_logp, float* d_out_entropy, float* d_out_lse,
                                     float* d_out_row_stats, int32_t row_stats_sum_p2, int32_t* d_error_flag,
                                     trlk_stream_t stream) {
    clear_error();
    if (int rc = check_view("logp_entropy_fwd: logits", d_logits, dtype, n_seq, rows_per_seq, vocab, seq_stride,
                            row_stride))
        return rc;
    TRLK_REQUIRE(n_index >= 0, TRLK_ERR_BAD_SHAPE, "logp_entropy_fwd: n_index must be >= 0 (got %d)", n_index);
    TRLK_REQUIRE(temperature > 0.f && temperature < INFINITY, TRLK_ERR_BAD_VALUE,
                 "logp_entropy_fwd: temperature must be positive and finite (got %g)", (double)temperature);
    const int64_t rows = n_seq * rows_per_seq;
    if (rows == 0) return TRLK_OK;
    TRLK_REQUIRE(n_index == 0 || (d_index != nullptr && d_out_logp != nullptr), TRLK_ERR_NULL_POINTER,
                 "logp_entropy_fwd: index / out_logp pointer is null");
    TRLK_REQUIRE(n_index > 0 || d_out_entropy != nullptr || d_out_lse != nullptr || d_out_row_stats != nullptr,
                 TRLK_ERR_NULL_POINTER, "logp_entropy_fwd: no output requested");
    TRLK_REQUIRE(d_out_row_stats == nullptr || vocab < (int64_t(1) << 24), TRLK_ERR_UNSUPPORTED,
                 "logp_entropy_fwd: row statistics need vocab < 2^24 (got %lld)", (long long)vocab);

    FwdArgs a{d_logits,    rows_per_seq, vocab,         seq_stride, row_stride,  d_index,
              n_index,     temperature,  d_row_mask,    d_out_logp, d_out_entropy, d_out_lse,
              d_out_row_stats, d_error_flag};
    const size_t es = elem_size(dtype);
    const bool vec = aligned16(d_logits, es, {seq_stride, row_stride}) && vocab % int64_t(16 / es) == 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)rows), block(kThreads);
    const int stats = d_out_row_stats == nullptr ? 0 : (row_stats_sum_p2 ? 2 : 1);
    // (One launch shape whatever the number of rows: 512 lanes x 2 loads per row is 5 % faster on launches that are a
    // single round of workgroups, but it sums a row in another order, and a row's log-prob must not depend on how many
    // other rows the launch holds -- a reference pass over part of a batch has to reproduce the policy pass bit for bit.)
#define TRLK_LAUNCH_FWD_VEC(DT, VEC)                                                           \
    if (stats == 2)                                                                            \
        hipLaunchKernelGGL((logp_entropy_fwd_kernel<DT, VEC, 2>), grid, block, 0, s, a);       \
    else if (stats == 1)                                                                       \
        hipLaunchKernelGGL((logp_entropy_fwd_kernel<DT, VEC, 1>), grid, block, 0, s, a);       \
    else                                                                                       \
        hipLaunchKernelGGL((logp_entropy_fwd_kernel<DT, VEC, 0>), grid, block, 0, s, a);
#define TRLK_LAUNCH_FWD(DT)                                                                    \
    if (vec) {                                                                                 \
        TRLK_LAUNCH_FWD_VEC(DT, true)                                                          \
    } else {                                                                                   \
        TRLK_LAUNCH_FWD_VEC(DT, false)                                                         \
    }
    if (dtype == TRLK_F32) {
        TRLK_LAUNCH_FWD(TRLK_F32)
    } else if (dtype == TRLK_BF16) {
        TRLK_LAUNCH_FWD(TRLK_BF16)
    } else {
        TRLK_LAUNCH_FWD(TRLK_F16)
    }
#undef TRLK_LAUNCH_FWD
#undef TRLK_LAUNCH_FWD_VEC
    return launch_status("logp_entropy_fwd");
}

extern "C" int trlk_logp_entropy_bwd(const void* d_logits, int dtype, int64_t n_seq, int64_t rows_per_seq,
                                     int64_t vocab, int64_t seq_stride, int64_t row_stride, const int64_t* d_index,
                                     int32_t n_index, float temperature, const float* d_lse, const float* d_entropy,
                                     const float* d_g_logp, const float* d_g_entropy, void* d_dlogits,
                                     int64_t out_rows_per_seq, int64_t out_row_offset, int64_t out_seq_stride,
                                     int64_t out_row_stride, trlk_stream_t stream) {
    clear_error();
    if (int rc = check_view("logp_entropy_bwd: logits", d_logits, dtype, n_seq, rows_per_seq, vocab, seq_stride,
                            row_stride))
        return rc;
    if (int rc = check_view("logp_entropy_bwd: dlogits", d_dlogits, dtype, n_seq, out_rows_per_seq, vocab,
                            out_seq_stride, out_row_stride))
        return rc;
    TRLK_REQUIRE(n_index >= 0 && n_index <= kMaxIndex, TRLK_ERR_UNSUPPORTED,
                 "logp_entropy_bwd: n_index must be in [0, %d] (got %d)", kMaxIndex, n_index);
    TRLK_REQUIRE(temperature > 0.f && temperature < INFINITY, TRLK_ERR_BAD_VALUE,
                 "logp_entropy_bwd: temperature must be positive and finite (got %g)", (double)temperature);
    TRLK_REQUIRE(out_row_offset >= 0 && out_row_offset + rows_per_seq <= out_rows_per_seq, TRLK_ERR_BAD_SHAPE,
                 "logp_entropy_bwd: input rows [%lld, %lld) do not fit the %lld output rows per sequence",
                 (long long)out_row_offset, (long long)(out_row_offset + rows_per_seq), (long long)out_rows_per_seq);
    const int64_t orows = n_seq * out_rows_per_seq;
    if (orows == 0) return TRLK_OK;
    if (n_seq * rows_per_seq > 0) {
        TRLK_REQUIRE(d_lse != nullptr, TRLK_ERR_NULL_POINTER, "logp_entropy_bwd: lse pointer is null");
        TRLK_REQUIRE(n_index == 0 || (d_index != nullptr && d_g_logp != nullptr), TRLK_ERR_NULL_POINTER,
                     "logp_entropy_bwd: index / g_logp pointer is null");
        TRLK_REQUIRE((d_g_entropy == nullptr) == (d_entropy == nullptr), TRLK_ERR_NULL_POINTER,
                     "logp_entropy_bwd: g_entropy and entropy must be given together");
        TRLK_REQUIRE(n_index > 0 || d_g_entropy != nullptr, TRLK_ERR_NULL_POINTER,
                     "logp_entropy_bwd: no upstream gradient given");
    }
    BwdArgs a{d_logits, rows_per_seq, vocab,    seq_stride,  row_stride, d_index,          n_index,
              temperature, d_lse,     d_entropy, d_g_logp,   d_g_entropy, d_dlogits,       out_rows_per_seq,
              out_row_offset, out_seq_stride, out_row_stride};
    const size_t es = elem_size(dtype);
    const bool vec = aligned16(d_logits, es, {seq_stride, row_stride}) &&
                     aligned16(d_dlogits, es, {out_seq_stride, out_row_stride}) && vocab % int64_t(16 / es) == 0;
    const bool has_h = d_g_entropy != nullptr;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t chunk = kChunkBytes / int64_t(es);
    const int64_t chunks_per_row = (vocab + chunk - 1) / chunk;
    TRLK_REQUIRE(orows * chunks_per_row < (int64_t(1) << 31) - 8, TRLK_ERR_BAD_SHAPE,
                 "logp_entropy_bwd: %lld rows x %lld chunks exceed the grid limit", (long long)orows,
                 (long long)chunks_per_row);
    a.total_chunks = orows * chunks_per_row;
    const dim3 grid((unsigned)(((a.total_chunks + 7) / 8) * 8)), block(kThreads);
    const int cpr = int(chunks_per_row);
#define TRLK_LAUNCH_BWD(DT)                                                                              \
    if (vec && has_h)                                                                                    \
        hipLaunchKernelGGL((logp_entropy_bwd_kernel<DT, true, true>), grid, block, 0, s, a, cpr);        \
    else if (vec)                                                                                        \
        hipLaunchKernelGGL((logp_entropy_bwd_kernel<DT, true, false>), grid, block, 0, s, a, cpr);       \
    else if (has_h)                                                                                      \
        hipLaunchKernelGGL((logp_entropy_bwd_kernel<DT, false, true>), grid, block, 0, s, a, cpr);       \
    else                                                                                                 \
        hipLaunchKernelGGL((logp_entropy_bwd_kernel<DT, false, false>), grid, block, 0, s, a, cpr);
    if (dtype == TRLK_F32) {
        TRLK_LAUNCH_BWD(TRLK_F32)
    } else if (dtype == TRLK_BF16) {
        TRLK_LAUNCH_BWD(TRLK_BF16)
    } else {
        TRLK_LAUNCH_BWD(TRLK_F16)
    }
#undef TRLK_LAUNCH_BWD
    return launch_status("logp_entropy_bwd");
}
