// What the memory system of this GPU sustains for the access shapes of the
// DeepSeek-V3 prefill step (4096 tokens, hidden 7168, top-8), with none of the
// library's routing in the way: the yardstick the library's kernels are measured
// against.
//
//   sweep      read-only, write-only and copy over 512 MiB; a write-only sweep
//              from 128 workgroups in 64 KiB pieces (few, long write streams are
//              the fastest writes seen here)
//   push       one workgroup of 448 threads per token: 32 bytes in per lane,
//              16 bytes out to each of 8 rows of 7168 bytes (the pack's shape,
//              stores at device scope as the library's); rows are a random
//              permutation of a dense buffer
//   gather     one wavefront per token and 1 KiB piece: 16 bytes from each of
//              8 rows of 14336 bytes, summed, 16 bytes out, non-temporal (the
//              combine's shape); once with the output predicated off
//   row copy   4096 rows picked through a table and written to rows picked
//              through another, a wavefront per row: rows of 7392 bytes (what a
//              rank's split recv moves) and of 14336 bytes (its combine-send)
//   1024       push and gather over the first 1024 tokens only
//   launches   what a dependent launch costs by itself: empty kernels of the library's launch shapes
//              (with 3.8 KB of arguments by value, as the library's) enqueued behind a kernel that
//              holds the queue for 20 ms, so that the host is ahead and the pace is the GPU's; and
//              what the events that a launch records at its own start and end read for an empty kernel
//
// Every kernel takes the number of its units and returns at once beyond it.
//
// What ran before matters, because it decides what the caches hold when the
// timed kernel starts: after a kernel that mostly reads (clean lines) the push
// is a fifth faster than after one that wrote 600 MiB (dirty lines to evict
// first).  So every timed launch follows a stated predecessor: the push follows
// the gather and the gather the push, as dispatch and combine alternate in a
// model; the sweeps follow a 600 MiB read.  The payload is random unless a
// line says otherwise: all-zero rows are written measurably faster, so constant
// data flatters a write-bound kernel.
//
// Usage: a2a_ceilings            (prints microseconds and GB/s, median of 20)
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <numeric>
#include <random>
#include <vector>

#define CHECK(call)                                                                                \
    do {                                                                                           \
        hipError_t err_ = (call);                                                                  \
        if (err_ != hipSuccess) {                                                                  \
            std::fprintf(stderr, "%s failed: %s (%s:%d)\n", #call, hipGetErrorString(err_), __FILE__, \
                         __LINE__);                                                                \
            std::exit(1);                                                                          \
        }                                                                                          \
    } while (0)

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr uint32_t kTokens = 4096, kTopk = 8, kHidden = 7168;
constexpr uint32_t kRows = kTokens * kTopk;
constexpr size_t kInRow = (size_t)kHidden * 2;    // bf16 token / expert output row
constexpr size_t kOutRow = kHidden;               // fp8 dispatched row

__global__ void read_sweep(const u32x4 *__restrict__ in, u32x4 *out, size_t n, uint32_t never) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    u32x4 acc = {0, 0, 0, 0};
    for (; i < n; i += stride) acc += __builtin_nontemporal_load(in + i);
    if (acc[0] == never) out[0] = acc;   // keeps the loads alive, never taken
}

__global__ void write_sweep(u32x4 *out, size_t n, uint32_t seed) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        const uint32_t v = (uint32_t)i * 2654435761u + seed;
        out[i] = u32x4{v, v ^ 0x9E3779B9u, v * 3u, v + 7u};
    }
}

__global__ void copy_sweep(const u32x4 *__restrict__ in, u32x4 *__restrict__ out, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) out[i] = __builtin_nontemporal_load(in + i);
}

// The pack without routing or arithmetic: the xor of two 16-byte halves stands
// for the quantised chunk (random in, random out; equal halves give zeros).
// Stores at device scope, as the library's pack.
__device__ __forceinline__ void store_sc1(u32x4 v, u32x4 *p) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}

__global__ __launch_bounds__(448) void push(const uint8_t *__restrict__ x, uint8_t *__restrict__ out,
                                            const uint32_t *__restrict__ slots, uint32_t tokens) {
    const uint32_t t = blockIdx.x, c = threadIdx.x;
    if (t >= tokens || c >= kHidden / 16) return;
    const u32x4 *p = reinterpret_cast<const u32x4 *>(x + (size_t)t * kInRow + (size_t)c * 32);
    const u32x4 a = __builtin_nontemporal_load(p), b = __builtin_nontemporal_load(p + 1);
    const u32x4 q = a ^ b;
#pragma unroll
    for (uint32_t k = 0; k < kTopk; ++k) {
        store_sc1(q, reinterpret_cast<u32x4 *>(out + (size_t)slots[t * kTopk + k] * kOutRow + (size_t)c * 16));
    }
}

// The combine without routing or arithmetic; a unit is one (token, 1 KiB piece).
// STORE = false predicates the output off (one value in 2^32 would store),
// leaving the reads alone.
constexpr uint32_t kPieces = (uint32_t)(kInRow / 1024);   // 14

template <bool STORE>
__global__ __launch_bounds__(64) void gather(const uint8_t *__restrict__ y, uint8_t *__restrict__ out,
                                             const uint32_t *__restrict__ slots, uint32_t units, uint32_t never) {
    const uint32_t unit = blockIdx.x;
    if (unit >= units) return;
    const uint32_t t = unit / kPieces, piece = unit - t * kPieces;
    const uint32_t c = piece * 64 + threadIdx.x;
    u32x4 v[kTopk];
#pragma unroll
    for (uint32_t k = 0; k < kTopk; ++k) {
        v[k] = __builtin_nontemporal_load(
            reinterpret_cast<const u32x4 *>(y + (size_t)slots[t * kTopk + k] * kInRow + (size_t)c * 16));
    }
    u32x4 acc = v[0];
#pragma unroll
    for (uint32_t k = 1; k < kTopk; ++k) acc += v[k];
    u32x4 *o = reinterpret_cast<u32x4 *>(out + (size_t)t * kInRow + (size_t)c * 16);
    if (STORE) {
        __builtin_nontemporal_store(acc, o);
    } else if (acc[0] == never) {
        *o = acc;
    }
}

// The split calls' row copies without their tables' meaning: row `from[i]` of `in` goes to row `to[i]`
// of `out`, one wavefront per row, eight 16-byte pieces per lane in flight.
__global__ __launch_bounds__(256) void row_copy(const uint8_t *__restrict__ in, uint8_t *__restrict__ out,
                                                const uint32_t *__restrict__ from, const uint32_t *__restrict__ to,
                                                uint32_t rows, uint32_t row_bytes) {
    const uint32_t row = blockIdx.x * 4 + threadIdx.x / 64, lane = threadIdx.x & 63;
    if (row >= rows) return;
    const u32x4 *src = reinterpret_cast<const u32x4 *>(in + (size_t)from[row] * row_bytes);
    u32x4 *dst = reinterpret_cast<u32x4 *>(out + (size_t)to[row] * row_bytes);
    const uint32_t chunks = row_bytes / 16;
    for (uint32_t c0 = 0; c0 < chunks; c0 += 512) {
        u32x4 v[8];
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u) {
            const uint32_t c = c0 + u * 64 + lane;
            if (c < chunks) v[u] = __builtin_nontemporal_load(src + c);
        }
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u) {
            const uint32_t c = c0 + u * 64 + lane;
            if (c < chunks) dst[c] = v[u];
        }
    }
}

// Write-only sweep in which each workgroup writes `chunk16` consecutive 16-byte pieces and then
// jumps by grid x chunk: the number of concurrent write streams and their length are the knobs.
// Few, long streams (128 workgroups x 64 KiB) are the fastest writes this GPU showed.
__global__ __launch_bounds__(256) void write_streams(u32x4 *out, size_t n16, uint32_t chunk16, uint32_t seed) {
    const size_t stride = (size_t)gridDim.x * chunk16;
    for (size_t base = (size_t)blockIdx.x * chunk16; base < n16; base += stride) {
        for (uint32_t i = threadIdx.x; i < chunk16; i += 256) {
            const size_t idx = base + i;
            if (idx < n16) {
                const uint32_t v = (uint32_t)idx * 2654435761u + seed;
                store_sc1(u32x4{v, v ^ 0x9E3779B9u, v * 3u, v + 7u}, out + idx);
            }
        }
    }
}

// The cost of a launch by itself.
struct Arguments {
    uint32_t w[960];   // 3840 bytes by value, about what the library's kernels take
};

__global__ void hold_queue(unsigned long long ticks, uint32_t *out) {   // wall_clock64 counts at 100 MHz
    const unsigned long long t0 = wall_clock64();
    while (wall_clock64() - t0 < ticks) {
    }
    if (threadIdx.x == 4096) out[0] = 1;
}

__global__ void empty(Arguments a, uint32_t *out, uint32_t never) {
    if (threadIdx.x == never) out[0] = a.w[never % 960];
}

struct Timer {
    hipStream_t stream;
    hipEvent_t start, stop;

    // Median over `reps` of: predecessor (untimed), then the timed launch.
    template <typename Before, typename Launch>
    float median_us(Before before, Launch launch, int reps = 20) {
        std::vector<float> us;
        for (int i = 0; i < reps + 4; ++i) {
            before();
            CHECK(hipEventRecord(start, stream));
            launch();
            CHECK(hipEventRecord(stop, stream));
            CHECK(hipEventSynchronize(stop));
            float ms = 0.0f;
            CHECK(hipEventElapsedTime(&ms, start, stop));
            if (i >= 4) us.push_back(ms * 1e3f);
        }
        CHECK(hipGetLastError());
        std::sort(us.begin(), us.end());
        return us[us.size() / 2];
    }
};

void report(const char *name, float us, double bytes) {
    std::printf("%-52s %7.1f us  %6.0f GB/s\n", name, us, bytes / (us * 1e-6) / 1e9);
    std::fflush(stdout);
}

void fill_random(void *device, size_t bytes, uint32_t seed) {
    std::vector<uint32_t> host(bytes / 4);
    uint32_t z = seed;
    for (auto &w : host) {
        z = z * 1664525u + 1013904223u;
        w = z ^ (z >> 15);
    }
    CHECK(hipMemcpy(device, host.data(), bytes, hipMemcpyHostToDevice));
}

}  // namespace

int main() {
    Timer timer;
    CHECK(hipStreamCreate(&timer.stream));
    CHECK(hipEventCreate(&timer.start));
    CHECK(hipEventCreate(&timer.stop));
    hipStream_t s = timer.stream;

    std::vector<uint32_t> slots(kRows);
    std::iota(slots.begin(), slots.end(), 0u);
    std::mt19937 rng(1);
    std::shuffle(slots.begin(), slots.end(), rng);
    uint32_t *d_slots;
    CHECK(hipMalloc(&d_slots, kRows * sizeof(uint32_t)));
    CHECK(hipMemcpy(d_slots, slots.data(), kRows * sizeof(uint32_t), hipMemcpyHostToDevice));

    uint8_t *x, *x_const, *dispatched, *y, *combined, *big_a, *big_b;
    const size_t sweep_bytes = (size_t)512 << 20;
    CHECK(hipMalloc(&x, kTokens * kInRow));
    CHECK(hipMalloc(&x_const, kTokens * kInRow));
    CHECK(hipMalloc(&dispatched, kRows * kOutRow));
    CHECK(hipMalloc(&y, kRows * kInRow));
    CHECK(hipMalloc(&combined, kTokens * kInRow));
    CHECK(hipMalloc(&big_a, sweep_bytes));
    CHECK(hipMalloc(&big_b, sweep_bytes));
    fill_random(x, kTokens * kInRow, 11);
    CHECK(hipMemset(x_const, 0x3c, kTokens * kInRow));
    fill_random(y, kRows * kInRow, 12);
    fill_random(big_a, sweep_bytes, 13);

    uint8_t *other;
    const size_t other_bytes = (size_t)600 << 20;
    CHECK(hipMalloc(&other, other_bytes));
    fill_random(other, other_bytes, 14);

    const size_t n16 = sweep_bytes / 16;
    auto read_other = [&] {
        hipLaunchKernelGGL(read_sweep, dim3(2048), dim3(256), 0, s, (const u32x4 *)other, (u32x4 *)big_b,
                           other_bytes / 16, 0x12345u);
    };
    auto fill_other = [&] {
        hipLaunchKernelGGL(write_sweep, dim3(512), dim3(256), 0, s, (u32x4 *)other, other_bytes / 16, 3u);
    };
    auto push_of = [&](const uint8_t *rows, uint32_t tokens) {
        return [=] { hipLaunchKernelGGL(push, dim3(tokens), dim3(448), 0, s, rows, dispatched, (const uint32_t *)d_slots, tokens); };
    };
    auto run_push = push_of(x, kTokens);
    auto run_push_zero = push_of(x_const, kTokens);
    auto gather_of = [&](uint32_t tokens, bool store) {
        return [=] {
            if (store) {
                hipLaunchKernelGGL(gather<true>, dim3(tokens * kPieces), dim3(64), 0, s, (const uint8_t *)y, combined,
                                   (const uint32_t *)d_slots, tokens * kPieces, 0x12345u);
            } else {
                hipLaunchKernelGGL(gather<false>, dim3(tokens * kPieces), dim3(64), 0, s, (const uint8_t *)y, combined,
                                   (const uint32_t *)d_slots, tokens * kPieces, 0x12345u);
            }
        };
    };
    auto run_gather = gather_of(kTokens, true);
    auto run_gather_reads = gather_of(kTokens, false);

    std::printf("after a 600 MiB read:\n");
    report("  read-only sweep, 512 MiB",
           timer.median_us(read_other, [&] { hipLaunchKernelGGL(read_sweep, dim3(2048), dim3(256), 0, s, (const u32x4 *)big_a, (u32x4 *)big_b, n16, 0x12345u); }),
           (double)sweep_bytes);
    report("  write-only sweep, 512 MiB, 512 workgroups",
           timer.median_us(read_other, [&] { hipLaunchKernelGGL(write_sweep, dim3(512), dim3(256), 0, s, (u32x4 *)big_b, n16, 5u); }),
           (double)sweep_bytes);
    report("  write-only sweep, 512 MiB, 4096 workgroups",
           timer.median_us(read_other, [&] { hipLaunchKernelGGL(write_sweep, dim3(4096), dim3(256), 0, s, (u32x4 *)big_b, n16, 5u); }),
           (double)sweep_bytes);
    report("  write-only, 128 workgroups x 64 KiB streams, sc1",
           timer.median_us(read_other, [&] { hipLaunchKernelGGL(write_streams, dim3(128), dim3(256), 0, s, (u32x4 *)big_b, n16, 4096u, 5u); }),
           (double)sweep_bytes);
    report("  copy, 512 MiB read + 512 MiB written",
           timer.median_us(read_other, [&] { hipLaunchKernelGGL(copy_sweep, dim3(2048), dim3(256), 0, s, (const u32x4 *)big_a, (u32x4 *)big_b, n16); }),
           2.0 * sweep_bytes);

    const double push_bytes = (double)kTokens * (kInRow + kTopk * kOutRow);
    const double gather_reads = (double)kTokens * kTopk * kInRow;
    const double gather_bytes = gather_reads + (double)kTokens * kInRow;
    std::printf("push and gather in turn, as dispatch and combine alternate:\n");
    report("  push (pack's shape), random payload", timer.median_us(run_gather, run_push), push_bytes);
    report("  push (pack's shape), all-zero rows written", timer.median_us(run_gather, run_push_zero), push_bytes);
    report("  gather (combine's shape)", timer.median_us(run_push, run_gather), gather_bytes);
    report("  gather, reads only (output predicated off)", timer.median_us(run_push, run_gather_reads), gather_reads);
    std::printf("after a 600 MiB fill (dirty caches):\n");
    report("  push (pack's shape), random payload", timer.median_us(fill_other, run_push), push_bytes);
    report("  gather (combine's shape)", timer.median_us(fill_other, run_gather), gather_bytes);
    report("  the gather's output alone, 56 MiB striped fill",
           timer.median_us(fill_other, [&] { hipLaunchKernelGGL(write_sweep, dim3(512), dim3(256), 0, s, (u32x4 *)combined, kTokens * kInRow / 16, 9u); }),
           (double)kTokens * kInRow);
    // The row copies of the split calls: 4096 rows (what one of 8 ranks receives of a 4096-token step),
    // sources and destinations each a random permutation of 4096 rows of a buffer that holds them all.
    std::printf("row copies of the split calls (4096 rows, a wavefront per row), after a 600 MiB read:\n");
    {
        std::vector<uint32_t> from(kTokens), to(kTokens);
        std::iota(from.begin(), from.end(), 0u);
        std::iota(to.begin(), to.end(), 0u);
        std::shuffle(from.begin(), from.end(), rng);
        std::shuffle(to.begin(), to.end(), rng);
        uint32_t *d_from, *d_to;
        CHECK(hipMalloc(&d_from, kTokens * sizeof(uint32_t)));
        CHECK(hipMalloc(&d_to, kTokens * sizeof(uint32_t)));
        CHECK(hipMemcpy(d_from, from.data(), kTokens * sizeof(uint32_t), hipMemcpyHostToDevice));
        CHECK(hipMemcpy(d_to, to.data(), kTokens * sizeof(uint32_t), hipMemcpyHostToDevice));
        for (uint32_t row_bytes : {7392u, 14336u}) {   // inside y (4096 x 8 rows of 14336 bytes) and big_b
            char name[96];
            std::snprintf(name, sizeof name, "  rows of %u bytes, read and written", row_bytes);
            report(name, timer.median_us(read_other, [&] {
                       hipLaunchKernelGGL(row_copy, dim3(kTokens / 4), dim3(256), 0, s, (const uint8_t *)y, big_b,
                                          (const uint32_t *)d_from, (const uint32_t *)d_to, kTokens, row_bytes);
                   }),
                   2.0 * kTokens * row_bytes);
        }
    }

    // The same two shapes at 1024 tokens (the Kimi-K2 mixed batch): the push is a single wave of
    // workgroups, so nothing overlaps its launch, its reads and its burst of writes.
    std::printf("at 1024 tokens, push and gather in turn:\n");
    constexpr uint32_t kFewTokens = 1024;
    auto few_push = push_of(x, kFewTokens);
    auto few_gather = gather_of(kFewTokens, true);
    report("  push, 1024 tokens", timer.median_us(few_gather, few_push),
           (double)kFewTokens * (kInRow + kTopk * kOutRow));
    report("  gather, 1024 tokens", timer.median_us(few_push, few_gather),
           (double)kFewTokens * (kTopk + 1) * kInRow);

    // What a launch costs by itself, for the launch shapes of the library's kernels.
    std::printf("empty kernels, 3.8 KB of arguments, 1000 dependent launches behind a kernel that holds the queue:\n");
    {
        Arguments a = {};
        uint32_t *flag = reinterpret_cast<uint32_t *>(combined);
        struct Shape { const char *name; uint32_t blocks, threads; };
        for (const Shape &sh : {Shape{"136 x 448 (128-token dispatch)", 136, 448}, Shape{"1792 x 64 (128-token gather)", 1792, 64},
                                Shape{"256 x 896 (1024-token dispatch)", 256, 896}, Shape{"4112 x 448 (4096-token pack)", 4112, 448},
                                Shape{"57344 x 64 (4096-token gather)", 57344, 64}}) {
            CHECK(hipStreamSynchronize(s));
            hipLaunchKernelGGL(hold_queue, dim3(1), dim3(64), 0, s, 2000000ull, flag);
            CHECK(hipEventRecord(timer.start, s));
            for (int i = 0; i < 1000; ++i) hipLaunchKernelGGL(empty, dim3(sh.blocks), dim3(sh.threads), 0, s, a, flag, 0xFFFFFu);
            CHECK(hipEventRecord(timer.stop, s));
            CHECK(hipEventSynchronize(timer.stop));
            float ms = 0.0f;
            CHECK(hipEventElapsedTime(&ms, timer.start, timer.stop));
            std::printf("  %-50s %7.2f us per launch\n", sh.name, ms);   // ms per 1000 launches = us per launch
        }
        hipEvent_t own_start, own_stop;
        CHECK(hipEventCreate(&own_start));
        CHECK(hipEventCreate(&own_stop));
        std::vector<float> own;
        for (int i = 0; i < 24; ++i) {
            hipExtLaunchKernelGGL(empty, dim3(136), dim3(448), 0, s, own_start, own_stop, 0, a, flag, 0xFFFFFu);
            CHECK(hipStreamSynchronize(s));
            float ms = 0.0f;
            CHECK(hipEventElapsedTime(&ms, own_start, own_stop));
            if (i >= 4) own.push_back(ms * 1e3f);
        }
        std::sort(own.begin(), own.end());
        std::printf("  %-50s %7.2f us\n", "between an empty launch's own start and stop events", own[own.size() / 2]);
    }
    return 0;
}
