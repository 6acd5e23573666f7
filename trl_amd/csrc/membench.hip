// What this GPU's memory system gives streaming kernels, by access pattern: the yardstick behind the roofline
// fractions quoted for the log-prob / gradient kernels.  Not part of libtrlk.so; `make -C trl_amd/csrc membench`
// builds build/membench, which allocates two 19.9 GB buffers (the logits / dlogits of the GRPO benchmark shape,
// 65536 rows of 151936 bf16) and prints one line per pattern.
//
// Patterns:
//   flat   consecutive workgroups on consecutive addresses; THREADS lanes, U 16-byte vectors per lane (a workgroup
//          covers THREADS * U * 16 bytes); read-only, write-only or copy; plain or non-temporal accesses
//   remap  the flat 4 KiB-per-workgroup pattern with consecutive workgroups S-way interleaved over the buffer, so
//          that S distant regions are written at the same time
//   row    one 1024-lane workgroup per 304 KB row, the row held in registers between its loads and its stores
//          (the access pattern of the single-pass GRPO kernel), every row or the benchmark's mask (48 % of the
//          rows are only zero-filled)
//   piece  the same with a row cut into 2 or 4 pieces, one workgroup per piece (several workgroups per CU at a
//          time, as a kernel whose workgroups exchange the row's statistics would run, without that exchange)
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <vector>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const u32x4 GIn;
typedef __attribute__((address_space(1))) u32x4 GOut;

#define CHECK(x)                                                                  \
    do {                                                                          \
        hipError_t e_ = (x);                                                      \
        if (e_ != hipSuccess) {                                                   \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
            exit(1);                                                              \
        }                                                                         \
    } while (0)

constexpr int kRowVec = 18992;  // 16-byte vectors per row
enum Kind { kRead = 0, kWrite = 1, kCopy = 2 };

template <int THREADS, int U, int KIND, bool NT>
__global__ __launch_bounds__(THREADS) void flat_kernel(const u32x4* __restrict__ in, u32x4* __restrict__ out, int64_t n,
                                                uint32_t never, int ways, int per_way) {
    int64_t blk = blockIdx.x;
    if (ways > 1) blk = (blk % ways) * int64_t(per_way) + blk / ways;
    const int64_t base = blk * THREADS * U;
    u32x4 q[U];
#pragma unroll
    for (int j = 0; j < U; ++j) {
        const int64_t v = base + j * THREADS + threadIdx.x;
        if (KIND == kWrite)
            q[j] = u32x4{never, 0u, 0u, 0u};
        else if (v < n)
            q[j] = NT ? __builtin_nontemporal_load(in + v) : in[v];
    }
    if (KIND == kRead) {
        uint32_t acc = 0;
#pragma unroll
        for (int j = 0; j < U; ++j) acc |= q[j].x & q[j].y & q[j].z & q[j].w;
        if (acc == never) out[base + threadIdx.x] = q[0];  // never true for the data used: keeps the loads alive
        return;
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
        const int64_t v = base + j * THREADS + threadIdx.x;
        if (v < n) {
            if (NT)
                __builtin_nontemporal_store(q[j], out + v);
            else
                out[v] = q[j];
        }
    }
}

// REGIONAL: consecutive workgroups go to the eight XCDs in turn; each XCD walks one contiguous eighth of the rows
// instead of every eighth row (the grid is a multiple of 8).
template <bool NT_LOAD, bool NT_STORE, bool REGIONAL = false>
__global__ __launch_bounds__(1024) void row_kernel(const u32x4* in, u32x4* out, const uint8_t* active) {
    constexpr int PER = (kRowVec + 1023) / 1024;
    const int tid = threadIdx.x;
    const int64_t row = REGIONAL ? int64_t(blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3) : int64_t(blockIdx.x);
    const u32x4* ip = in + row * kRowVec;
    u32x4* op = out + row * kRowVec;
    if (!active[row]) {
        const u32x4 z = {0u, 0u, 0u, 0u};
        for (int v = tid; v < kRowVec; v += 1024) __builtin_nontemporal_store(z, op + v);
        return;
    }
    u32x4 q[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        GIn* vj = (GIn*)ip + j * 1024;
        asm volatile("" : "+s"(vj));
        const int tj = (j + 1) * 1024 > kRowVec ? min(tid, kRowVec - 1 - j * 1024) : tid;
        q[j] = NT_LOAD ? __builtin_nontemporal_load(vj + tj) : vj[tj];
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) asm volatile("" : "+v"(q[j]));
#pragma unroll
    for (int j = 0; j < PER; ++j)
        if (j * 1024 + tid < kRowVec) {
            GOut* oj = (GOut*)op + j * 1024;
            asm volatile("" : "+s"(oj));
            if (NT_STORE)
                __builtin_nontemporal_store(q[j], oj + tid);
            else
                oj[tid] = q[j];
        }
}

// GROUP workgroups of one XCD share GROUP neighbouring rows: each takes the same slice (a GROUP-th of the row, at most
// 1024 vectors) of every one of them, so that a row is read and written by GROUP compute units at the same time and
// a workgroup still holds a row's worth of vectors.  (What a kernel that keeps its rows on chip would look like to
// the memory if the rows were spread over the compute units of an XCD; the statistics such a kernel needs per row
// would have to be exchanged between the workgroups, which this copy does not do.)
template <int GROUP>
__global__ __launch_bounds__(1024) void slice_kernel(const u32x4* in, u32x4* out, const uint8_t* active, int64_t rows_per_xcd) {
    constexpr int kSliceVec = (kRowVec + GROUP - 1) / GROUP;
    static_assert(kSliceVec <= 1024, "a slice is at most one vector per lane");
    const int tid = threadIdx.x;
    const int64_t slot = blockIdx.x >> 3;
    const int64_t group = slot / GROUP;
    const int slice = int(slot % GROUP);
    const int64_t row0 = int64_t(blockIdx.x & 7) * rows_per_xcd + group * GROUP;
    if (group * GROUP + GROUP > rows_per_xcd) return;  // (the last few rows of a region are left out of this test)
    const int v = slice * kSliceVec + tid;
    const bool mine = tid < kSliceVec && v < kRowVec;
    u32x4 q[GROUP];
#pragma unroll
    for (int j = 0; j < GROUP; ++j)
        if (mine && active[row0 + j]) q[j] = in[(row0 + j) * kRowVec + v];
#pragma unroll
    for (int j = 0; j < GROUP; ++j) asm volatile("" : "+v"(q[j]));
    const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < GROUP; ++j)
        if (mine) __builtin_nontemporal_store(active[row0 + j] ? q[j] : z, out + (row0 + j) * kRowVec + v);
}

// A workgroup takes RUN consecutive rows and refills every register with the next row's vector as soon as it has stored
// the current row's: a compute unit then reads and writes all the time instead of a row's worth of loads followed by a
// row's worth of stores, and the next row's load latency hides behind the current row's stores.
template <int RUN>
__global__ __launch_bounds__(1024) void row_run_kernel(const u32x4* in, u32x4* out, const uint8_t* active, int64_t rows_per_xcd) {
    constexpr int PER = (kRowVec + 1023) / 1024;
    const int tid = threadIdx.x;
    const int64_t row0 = int64_t(blockIdx.x & 7) * rows_per_xcd + int64_t(blockIdx.x >> 3) * RUN;
    u32x4 q[PER];
    // the flags of the whole run first: a flag loaded inside the loop would wait for everything in flight
    uint64_t flags = 0;
    for (int i = 0; i < RUN; ++i) flags |= uint64_t(active[row0 + i] != 0) << i;
    flags = __builtin_amdgcn_readfirstlane(uint32_t(flags)) | uint64_t(__builtin_amdgcn_readfirstlane(uint32_t(flags >> 32))) << 32;
    bool have = flags & 1;
    if (have) {
#pragma unroll
        for (int j = 0; j < PER; ++j)
            if (j * 1024 + tid < kRowVec) q[j] = in[row0 * kRowVec + j * 1024 + tid];
    }
    const u32x4 z = {0u, 0u, 0u, 0u};
    // (short runs are unrolled: across a loop's back edge the compiler waits for everything in flight, the stores'
    // acknowledgements included, and the straight-line form waits for exactly the load it stores next)
#pragma unroll(RUN <= 8 ? RUN : 1)
    for (int i = 0; i < RUN; ++i) {
        const int64_t row = row0 + i;
        const bool next = i + 1 < RUN && ((flags >> (i + 1)) & 1);
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            if (j * 1024 + tid < kRowVec) {
                __builtin_nontemporal_store(have ? q[j] : z, out + row * kRowVec + j * 1024 + tid);
                if (next) q[j] = in[(row + 1) * kRowVec + j * 1024 + tid];
            }
        }
        have = next;
    }
}

template <int THREADS, int PARTS>
__global__ __launch_bounds__(THREADS) void piece_kernel(const u32x4* in, u32x4* out, const uint8_t* active) {
    constexpr int kPieceVec = (kRowVec + PARTS - 1) / PARTS;
    constexpr int PER = (kPieceVec + THREADS - 1) / THREADS;
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x / PARTS;
    const int v0 = int(blockIdx.x % PARTS) * kPieceVec, nv = min(v0 + kPieceVec, kRowVec) - v0;
    const u32x4* ip = in + row * kRowVec + v0;
    u32x4* op = out + row * kRowVec + v0;
    if (!active[row]) {
        const u32x4 z = {0u, 0u, 0u, 0u};
        for (int v = tid; v < nv; v += THREADS) __builtin_nontemporal_store(z, op + v);
        return;
    }
    u32x4 q[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        GIn* vj = (GIn*)ip + j * THREADS;
        asm volatile("" : "+s"(vj));
        if (j * THREADS < nv) q[j] = vj[max(min(tid, nv - 1 - j * THREADS), 0)];
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) asm volatile("" : "+v"(q[j]));
#pragma unroll
    for (int j = 0; j < PER; ++j)
        if (j * THREADS + tid < nv) {
            GOut* oj = (GOut*)op + j * THREADS;
            asm volatile("" : "+s"(oj));
            __builtin_nontemporal_store(q[j], oj + tid);
        }
}

int main() {
    const int B = 64, T = 1024;
    const int64_t rows = int64_t(B) * T, n = rows * kRowVec;
    const size_t bytes = size_t(n) * 16;
    u32x4 *in, *out;
    uint8_t* act_d;
    CHECK(hipMalloc(&in, bytes));
    CHECK(hipMalloc(&out, bytes));
    CHECK(hipMalloc(&act_d, rows));
    CHECK(hipMemset(in, 1, bytes));
    CHECK(hipMemset(out, 0, bytes));
    std::vector<uint8_t> act(rows), ones(rows, 1);
    srand(1);
    int64_t n_act = 0;
    for (int b = 0; b < B; ++b) {
        const int len = 64 + rand() % (T - 64 + 1);
        for (int t = 0; t < T; ++t) n_act += (act[b * T + t] = t < len);
    }
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    auto run = [&](const char* name, double moved, auto launch) {
        launch();
        CHECK(hipDeviceSynchronize());
        CHECK(hipEventRecord(e0));
        const int reps = 5;
        for (int i = 0; i < reps; ++i) launch();
        CHECK(hipEventRecord(e1));
        CHECK(hipEventSynchronize(e1));
        float ms;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        ms /= reps;
        printf("%-52s %7.3f ms  %5.2f TB/s  %4.1f %% of 8 TB/s\n", name, ms, moved / ms / 1e9, moved / ms / 1e9 / 8.0 * 100);
        fflush(stdout);
    };
#define FLAT(TH, U, KIND, NT, WAYS)                                                                                     \
    {                                                                                                                   \
        const unsigned nb = unsigned(n / (TH * U));                                                                     \
        run("flat " #KIND " threads=" #TH " vectors/lane=" #U " nt=" #NT " ways=" #WAYS, (KIND == kCopy ? 2.0 : 1.0) * nb * TH * U * 16, \
            [&] { hipLaunchKernelGGL((flat_kernel<TH, U, KIND, NT>), dim3(nb), dim3(TH), 0, 0, in, out, n, 0xdeadbeefu, WAYS, int(nb / WAYS)); }); \
    }
    FLAT(256, 1, kRead, false, 1) FLAT(256, 4, kRead, false, 1) FLAT(256, 4, kRead, true, 1) FLAT(1024, 19, kRead, true, 1)
    FLAT(256, 1, kWrite, true, 1) FLAT(256, 2, kWrite, true, 1) FLAT(256, 4, kWrite, true, 1) FLAT(1024, 1, kWrite, true, 1)
    FLAT(1024, 19, kWrite, true, 1)
    FLAT(64, 1, kCopy, true, 1) FLAT(256, 1, kCopy, false, 1) FLAT(256, 1, kCopy, true, 1) FLAT(256, 2, kCopy, true, 1)
    FLAT(256, 4, kCopy, true, 1) FLAT(256, 8, kCopy, true, 1) FLAT(1024, 1, kCopy, true, 1) FLAT(1024, 19, kCopy, true, 1)
    FLAT(256, 1, kWrite, true, 8) FLAT(256, 1, kWrite, true, 64) FLAT(256, 1, kWrite, true, 512)
    FLAT(256, 1, kCopy, true, 8) FLAT(256, 1, kCopy, true, 64) FLAT(256, 1, kCopy, true, 512)
    const double row_bytes = kRowVec * 16.0;
    for (int masked = 0; masked < 2; ++masked) {
        CHECK(hipMemcpy(act_d, masked ? act.data() : ones.data(), rows, hipMemcpyHostToDevice));
        const double moved = masked ? (n_act * 2 + (rows - n_act)) * row_bytes : 2.0 * rows * row_bytes;
        run(masked ? "row in registers, benchmark mask, plain/plain" : "row in registers, every row, plain/plain", moved,
            [&] { hipLaunchKernelGGL((row_kernel<false, false>), dim3(unsigned(rows)), dim3(1024), 0, 0, in, out, act_d); });
        run(masked ? "row in registers, benchmark mask, plain/nt" : "row in registers, every row, plain/nt", moved,
            [&] { hipLaunchKernelGGL((row_kernel<false, true>), dim3(unsigned(rows)), dim3(1024), 0, 0, in, out, act_d); });
        run(masked ? "row in registers, benchmark mask, nt/nt" : "row in registers, every row, nt/nt", moved,
            [&] { hipLaunchKernelGGL((row_kernel<true, true>), dim3(unsigned(rows)), dim3(1024), 0, 0, in, out, act_d); });
        run(masked ? "row in registers, one region of rows per XCD, benchmark mask, plain/nt"
                   : "row in registers, one region of rows per XCD, every row, plain/nt", moved,
            [&] { hipLaunchKernelGGL((row_kernel<false, true, true>), dim3(unsigned(rows)), dim3(1024), 0, 0, in, out, act_d); });
        {
            constexpr int G = 19;
            const int64_t per_xcd = rows / 8, groups = per_xcd / G;
            int64_t act_in = 0, all_in = 0;  // the rows the grouped kernel covers
            for (int x = 0; x < 8; ++x)
                for (int64_t r = 0; r < groups * G; ++r) {
                    act_in += masked ? act[x * per_xcd + r] : 1;
                    ++all_in;
                }
            const double moved_g = (act_in * 2 + (all_in - act_in)) * row_bytes;
            run(masked ? "19 rows sliced over 19 workgroups of an XCD, benchmark mask" : "19 rows sliced over 19 workgroups of an XCD, every row",
                moved_g, [&] { hipLaunchKernelGGL((slice_kernel<G>), dim3(unsigned(8 * groups * G)), dim3(1024), 0, 0, in, out, act_d, per_xcd); });
        }
        run(masked ? "runs of 4 rows per workgroup, refilled while storing, benchmark mask" : "runs of 4 rows per workgroup, refilled while storing, every row",
            moved, [&] { hipLaunchKernelGGL((row_run_kernel<4>), dim3(unsigned(rows / 4)), dim3(1024), 0, 0, in, out, act_d, rows / 8); });
        run(masked ? "runs of 8 rows per workgroup, refilled while storing, benchmark mask" : "runs of 8 rows per workgroup, refilled while storing, every row",
            moved, [&] { hipLaunchKernelGGL((row_run_kernel<8>), dim3(unsigned(rows / 8)), dim3(1024), 0, 0, in, out, act_d, rows / 8); });
        run(masked ? "runs of 64 rows per workgroup, refilled while storing, benchmark mask" : "runs of 64 rows per workgroup, refilled while storing, every row",
            moved, [&] { hipLaunchKernelGGL((row_run_kernel<64>), dim3(unsigned(rows / 64)), dim3(1024), 0, 0, in, out, act_d, rows / 8); });
        run(masked ? "2 pieces of 1024 lanes, benchmark mask, plain/nt" : "2 pieces of 1024 lanes, every row, plain/nt", moved,
            [&] { hipLaunchKernelGGL((piece_kernel<1024, 2>), dim3(unsigned(rows * 2)), dim3(1024), 0, 0, in, out, act_d); });
        run(masked ? "2 pieces of 512 lanes, benchmark mask, plain/nt" : "2 pieces of 512 lanes, every row, plain/nt", moved,
            [&] { hipLaunchKernelGGL((piece_kernel<512, 2>), dim3(unsigned(rows * 2)), dim3(512), 0, 0, in, out, act_d); });
        run(masked ? "4 pieces of 1024 lanes, benchmark mask, plain/nt" : "4 pieces of 1024 lanes, every row, plain/nt", moved,
            [&] { hipLaunchKernelGGL((piece_kernel<1024, 4>), dim3(unsigned(rows * 4)), dim3(1024), 0, 0, in, out, act_d); });
        run(masked ? "4 pieces of 256 lanes, benchmark mask, plain/nt" : "4 pieces of 256 lanes, every row, plain/nt", moved,
            [&] { hipLaunchKernelGGL((piece_kernel<256, 4>), dim3(unsigned(rows * 4)), dim3(256), 0, 0, in, out, act_d); });
    }
    run("hipMemcpyAsync device to device", 2.0 * bytes, [&] { CHECK(hipMemcpyAsync(out, in, bytes, hipMemcpyDeviceToDevice, 0)); });
    return 0;
}
