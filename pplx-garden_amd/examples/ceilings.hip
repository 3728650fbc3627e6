// What the memory system of this GPU sustains for the access shapes of the
// DeepSeek-V3 prefill step (4096 tokens, hidden 7168, top-8), with none of the
// library's routing in the way: the yardstick the pack and the gather kernels
// are measured against.
//
//   sweep      read-only, write-only and copy over 512 MiB
//   push       one workgroup of 448 threads per token: 32 bytes in per lane,
//              16 bytes out to each of 8 rows of 7168 bytes (the pack's shape);
//              rows are a random permutation of a dense buffer
//   gather     one wavefront per token and 1 KiB piece: 16 bytes from each of
//              8 rows of 14336 bytes, summed, 16 bytes out (the combine's shape)
//   variants   the same gather with its output written through every cache
//              policy the store instruction has, with cached loads, and in
//              three shapes meant to make the writes overlap the reads (a
//              persistent wavefront that asks for the next unit's rows before
//              it stores the current one; a wavefront per workgroup that only
//              stores what three others hand it through LDS; persistent
//              workgroups that collect 16 to 64 KiB of output in LDS and write
//              it in one burst); and the push with the same store policies and
//              with half a token per workgroup
//   1024       push and gather over the first 1024 tokens only
//              the gather with fewer wavefronts per compute unit, and with the
//              workgroup -> unit mapping arranged by XCD (a token per XCD; a
//              contiguous eighth of the tokens per XCD);
//              and the push with its store policies, by XCD ranges, from 256 persistent
//              workgroups (fewer concurrent writers), and turned round into a
//              pull by destination row (sequential writes, input read 8 times)
//   streams    a write-only sweep from 128 workgroups in 64 KiB pieces: few, long
//              write streams are the fastest writes seen here (more workgroups
//              or shorter pieces fall back to the plain sweep's rate)
//
// Every gather variant takes the number of units (token x 1 KiB piece) and
// returns at once for a unit beyond it; the host derives each grid from the
// unit count in one place (launch_units) and refuses a grid that would cover
// more than the buffers hold.
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
__global__ __launch_bounds__(448) void push(const uint8_t *__restrict__ x, uint8_t *__restrict__ out,
                                            const uint32_t *__restrict__ slots) {
    const uint32_t t = blockIdx.x, c = threadIdx.x;
    if (t >= kTokens || c >= kHidden / 16) return;
    const u32x4 *p = reinterpret_cast<const u32x4 *>(x + (size_t)t * kInRow + (size_t)c * 32);
    const u32x4 a = __builtin_nontemporal_load(p), b = __builtin_nontemporal_load(p + 1);
    const u32x4 q = a ^ b;
#pragma unroll
    for (uint32_t k = 0; k < kTopk; ++k) {
        *reinterpret_cast<u32x4 *>(out + (size_t)slots[t * kTopk + k] * kOutRow + (size_t)c * 16) = q;
    }
}

// The combine without routing or arithmetic.  STORE = false predicates the
// output off (one value in 2^32 would store), leaving the reads alone.
template <bool STORE>
__global__ __launch_bounds__(64) void gather(const uint8_t *__restrict__ y, uint8_t *__restrict__ out,
                                             const uint32_t *__restrict__ slots, uint32_t never) {
    const uint32_t t = blockIdx.x / 14, piece = blockIdx.x % 14;
    if (t >= kTokens) return;
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


// ---- variants of the gather; a unit is one (token, 1 KiB piece) ----
constexpr uint32_t kPieces = (uint32_t)(kInRow / 1024);   // 14
constexpr uint32_t kUnits = kTokens * kPieces;

__device__ __forceinline__ void load_unit(u32x4 (&v)[kTopk], const uint8_t *y, const uint32_t *slots, uint32_t unit) {
    const uint32_t t = unit / kPieces, piece = unit - t * kPieces;
    const uint32_t c = piece * 64 + (threadIdx.x & 63);
#pragma unroll
    for (uint32_t k = 0; k < kTopk; ++k) {
        v[k] = __builtin_nontemporal_load(
            reinterpret_cast<const u32x4 *>(y + (size_t)slots[t * kTopk + k] * kInRow + (size_t)c * 16));
    }
}

__device__ __forceinline__ u32x4 sum_unit(const u32x4 (&v)[kTopk]) {
    u32x4 acc = v[0];
#pragma unroll
    for (uint32_t k = 1; k < kTopk; ++k) acc += v[k];
    return acc;
}

__device__ __forceinline__ u32x4 *out_of_unit(uint8_t *out, uint32_t unit) {
    const uint32_t t = unit / kPieces, piece = unit - t * kPieces;
    return reinterpret_cast<u32x4 *>(out + (size_t)t * kInRow + (size_t)(piece * 64 + (threadIdx.x & 63)) * 16);
}

// Cache policy of the 16-byte output store.
enum StorePolicy { kStoreNt, kStorePlain, kStoreSc0Sc1, kStoreSc1, kStoreSc0, kStoreSc0Sc1Nt };

template <int POLICY>
__device__ __forceinline__ void store_unit(u32x4 v, u32x4 *p) {
    if (POLICY == kStoreNt) {
        __builtin_nontemporal_store(v, p);
    } else if (POLICY == kStorePlain) {
        *p = v;
    } else if (POLICY == kStoreSc0Sc1) {
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(p), "v"(v) : "memory");
    } else if (POLICY == kStoreSc1) {
        asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
    } else if (POLICY == kStoreSc0) {
        asm volatile("global_store_dwordx4 %0, %1, off sc0" ::"v"(p), "v"(v) : "memory");
    } else {
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt" ::"v"(p), "v"(v) : "memory");
    }
}

// One unit per wavefront, as `gather`, with the store policy a parameter.
template <int POLICY>
__global__ __launch_bounds__(64) void gather_policy(const uint8_t *__restrict__ y, uint8_t *__restrict__ out,
                                                    const uint32_t *__restrict__ slots, uint32_t units) {
    const uint32_t unit = blockIdx.x;
    if (unit >= units) return;
    u32x4 v[kTopk];
    load_unit(v, y, slots, unit);
    store_unit<POLICY>(sum_unit(v), out_of_unit(out, unit));
}

// Which XCD works on what: workgroups are dealt to the 8 XCDs round-robin (workgroup b runs on XCD
// b % 8), so `unit = b` spreads every token's pieces over all XCDs and the output advances as ONE
// front.  MAP 1 keeps the 14 pieces of a token on one XCD (tokens dealt round-robin); MAP 2 gives each
// XCD a contiguous eighth of the tokens (8 separate output fronts).
template <int MAP>
__global__ __launch_bounds__(64) void gather_mapped(const uint8_t *__restrict__ y, uint8_t *__restrict__ out,
                                                    const uint32_t *__restrict__ slots, uint32_t units) {
    const uint32_t b = blockIdx.x;
    if (b >= units) return;
    const uint32_t xcd = b & 7, i = b >> 3;
    const uint32_t unit = MAP == 1 ? ((i / kPieces) * 8 + xcd) * kPieces + i % kPieces : xcd * (kUnits / 8) + i;
    if (unit >= units) return;
    u32x4 v[kTopk];
    load_unit(v, y, slots, unit);
    store_unit<kStoreNt>(sum_unit(v), out_of_unit(out, unit));
}

// Ordinary (cached) loads instead of non-temporal ones.
__global__ __launch_bounds__(64) void gather_cached_loads(const uint8_t *__restrict__ y, uint8_t *__restrict__ out,
                                                          const uint32_t *__restrict__ slots, uint32_t units) {
    const uint32_t unit = blockIdx.x;
    if (unit >= units) return;
    const uint32_t t = unit / kPieces, piece = unit - t * kPieces, c = piece * 64 + threadIdx.x;
    u32x4 v[kTopk];
#pragma unroll
    for (uint32_t k = 0; k < kTopk; ++k) {
        v[k] = *reinterpret_cast<const u32x4 *>(y + (size_t)slots[t * kTopk + k] * kInRow + (size_t)c * 16);
    }
    __builtin_nontemporal_store(sum_unit(v), out_of_unit(out, unit));
}

// Persistent wavefronts, software-pipelined: the rows of the next unit are asked
// for before the current unit is stored.
__global__ __launch_bounds__(64) void gather_pipelined(const uint8_t *__restrict__ y, uint8_t *__restrict__ out,
                                                       const uint32_t *__restrict__ slots, uint32_t units) {
    const uint32_t stride = gridDim.x;
    uint32_t unit = blockIdx.x;
    if (unit >= units) return;
    u32x4 cur[kTopk], nxt[kTopk];
    load_unit(cur, y, slots, unit);
    while (true) {
        const uint32_t next = unit + stride;
        const bool more = next < units;
        if (more) load_unit(nxt, y, slots, next);
        __builtin_nontemporal_store(sum_unit(cur), out_of_unit(out, unit));
        if (!more) break;
        for (uint32_t k = 0; k < kTopk; ++k) cur[k] = nxt[k];
        unit = next;
    }
}

// Three wavefronts gather; the fourth only stores what they hand it through LDS.
__global__ __launch_bounds__(256) void gather_store_wave(const uint8_t *__restrict__ y, uint8_t *__restrict__ out,
                                                         const uint32_t *__restrict__ slots, uint32_t units) {
    __shared__ u32x4 stage[3][64];
    const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x & 63;
    const uint32_t first = blockIdx.x * 3;
    if (wave < 3 && first + wave < units) {
        u32x4 v[kTopk];
        load_unit(v, y, slots, first + wave);
        stage[wave][lane] = sum_unit(v);
    }
    __syncthreads();
    if (wave == 3) {
#pragma unroll
        for (uint32_t w = 0; w < 3; ++w) {
            if (first + w < units) __builtin_nontemporal_store(stage[w][lane], out_of_unit(out, first + w));
        }
    }
}

// Persistent workgroups of 16 wavefronts collect ROUNDS x 16 KiB of output in LDS,
// then write it in one burst.
template <int ROUNDS>
__global__ __launch_bounds__(1024) void gather_bursts(const uint8_t *__restrict__ y, uint8_t *__restrict__ out,
                                                      const uint32_t *__restrict__ slots, uint32_t units) {
    extern __shared__ u32x4 collected[];   // [ROUNDS][16][64]
    const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x & 63;
    const uint32_t per_group = 16 * ROUNDS;
    for (uint32_t first = blockIdx.x * per_group; first < units; first += gridDim.x * per_group) {
        for (uint32_t r = 0; r < ROUNDS; ++r) {
            const uint32_t unit = first + r * 16 + wave;
            if (unit < units) {
                u32x4 v[kTopk];
                load_unit(v, y, slots, unit);
                collected[(r * 16 + wave) * 64 + lane] = sum_unit(v);
            }
        }
        __syncthreads();
        for (uint32_t r = 0; r < ROUNDS; ++r) {
            const uint32_t unit = first + r * 16 + wave;
            if (unit < units) __builtin_nontemporal_store(collected[(r * 16 + wave) * 64 + lane], out_of_unit(out, unit));
        }
        __syncthreads();
    }
}

// The push with the cache policy of its stores a parameter, and HALF of a token per
// workgroup when SPLIT is set (twice the workgroups, 224 of 256 threads active).
template <int POLICY, bool SPLIT>
__global__ __launch_bounds__(SPLIT ? 256 : 448) void push_policy(const uint8_t *__restrict__ x,
                                                                uint8_t *__restrict__ out,
                                                                const uint32_t *__restrict__ slots, uint32_t tokens) {
    const uint32_t t = SPLIT ? blockIdx.x / 2 : blockIdx.x;
    const uint32_t c = SPLIT ? (blockIdx.x & 1) * 224 + threadIdx.x : threadIdx.x;
    if (t >= tokens || c >= kHidden / 16 || (SPLIT && threadIdx.x >= 224)) return;
    const u32x4 *p = reinterpret_cast<const u32x4 *>(x + (size_t)t * kInRow + (size_t)c * 32);
    const u32x4 a = __builtin_nontemporal_load(p), b = __builtin_nontemporal_load(p + 1);
    const u32x4 q = a ^ b;
#pragma unroll
    for (uint32_t k = 0; k < kTopk; ++k) {
        store_unit<POLICY>(q, reinterpret_cast<u32x4 *>(out + (size_t)slots[t * kTopk + k] * kOutRow + (size_t)c * 16));
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
                store_unit<kStoreSc1>(u32x4{v, v ^ 0x9E3779B9u, v * 3u, v + 7u}, out + idx);
            }
        }
    }
}

// The push from persistent workgroups: workgroup b takes tokens b, b + grid, ... (a throttled
// number of writers instead of one workgroup per token).
__global__ __launch_bounds__(448) void push_persistent(const uint8_t *__restrict__ x, uint8_t *__restrict__ out,
                                                       const uint32_t *__restrict__ slots, uint32_t tokens) {
    const uint32_t c = threadIdx.x;
    if (c >= kHidden / 16) return;
    for (uint32_t t = blockIdx.x; t < tokens; t += gridDim.x) {
        const u32x4 *p = reinterpret_cast<const u32x4 *>(x + (size_t)t * kInRow + (size_t)c * 32);
        const u32x4 q = __builtin_nontemporal_load(p) ^ __builtin_nontemporal_load(p + 1);
#pragma unroll
        for (uint32_t k = 0; k < kTopk; ++k) {
            store_unit<kStoreSc1>(q, reinterpret_cast<u32x4 *>(out + (size_t)slots[t * kTopk + k] * kOutRow + (size_t)c * 16));
        }
    }
}

// The push with each XCD working through a contiguous eighth of the tokens.
__global__ __launch_bounds__(448) void push_xcd_ranges(const uint8_t *__restrict__ x, uint8_t *__restrict__ out,
                                                       const uint32_t *__restrict__ slots, uint32_t tokens) {
    const uint32_t b = blockIdx.x, c = threadIdx.x;
    const uint32_t t = (b & 7) * (tokens / 8) + (b >> 3);
    if (b >= tokens || t >= tokens || c >= kHidden / 16) return;
    const u32x4 *p = reinterpret_cast<const u32x4 *>(x + (size_t)t * kInRow + (size_t)c * 32);
    const u32x4 q = __builtin_nontemporal_load(p) ^ __builtin_nontemporal_load(p + 1);
#pragma unroll
    for (uint32_t k = 0; k < kTopk; ++k) {
        store_unit<kStoreSc1>(q, reinterpret_cast<u32x4 *>(out + (size_t)slots[t * kTopk + k] * kOutRow + (size_t)c * 16));
    }
}

// The pack turned round: one workgroup per DESTINATION row, rows in order, so the writes are one
// sequential stream; the price is that every token's input is read once per route (8 times).
__global__ __launch_bounds__(448) void pull_by_row(const uint8_t *__restrict__ x, uint8_t *__restrict__ out,
                                                   const uint32_t *__restrict__ token_of_row, uint32_t rows) {
    const uint32_t r = blockIdx.x, c = threadIdx.x;
    if (r >= rows || c >= kHidden / 16) return;
    const u32x4 *p = reinterpret_cast<const u32x4 *>(x + (size_t)token_of_row[r] * kInRow + (size_t)c * 32);
    store_unit<kStoreSc1>(p[0] ^ p[1], reinterpret_cast<u32x4 *>(out + (size_t)r * kOutRow + (size_t)c * 16));
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
    std::vector<uint32_t> token_of_row(kRows);
    for (uint32_t i = 0; i < kRows; ++i) token_of_row[slots[i]] = i / kTopk;
    uint32_t *d_token_of_row;
    CHECK(hipMalloc(&d_token_of_row, kRows * sizeof(uint32_t)));
    CHECK(hipMemcpy(d_token_of_row, token_of_row.data(), kRows * sizeof(uint32_t), hipMemcpyHostToDevice));

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
    auto run_push = [&] { hipLaunchKernelGGL(push, dim3(kTokens), dim3(448), 0, s, x, dispatched, d_slots); };
    auto run_push_zero = [&] { hipLaunchKernelGGL(push, dim3(kTokens), dim3(448), 0, s, x_const, dispatched, d_slots); };
    auto run_gather = [&] {
        hipLaunchKernelGGL(gather<true>, dim3(kTokens * 14), dim3(64), 0, s, y, combined, d_slots, 0x12345u);
    };
    auto run_gather_reads = [&] {
        hipLaunchKernelGGL(gather<false>, dim3(kTokens * 14), dim3(64), 0, s, y, combined, d_slots, 0x12345u);
    };

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
    // Variants of the gather.  Every launch goes through launch_units: the grid comes from the unit
    // count, and a grid whose last workgroup would start beyond the units is refused on the host
    // (the kernels also return for such a unit).
    std::printf("variants of the gather (after a push):\n");
    auto launch_units = [&](auto kernel, uint32_t blocks, uint32_t threads, size_t lds, uint32_t units_per_block) {
        if (blocks == 0 || (uint64_t)(blocks - 1) * units_per_block >= kUnits || lds > 64 * 1024) {
            std::fprintf(stderr, "refusing a grid of %u workgroups x %u units for %u units\n", blocks,
                         units_per_block, kUnits);
            std::exit(2);
        }
        hipLaunchKernelGGL(kernel, dim3(blocks), dim3(threads), lds, s, (const uint8_t *)y, combined,
                           (const uint32_t *)d_slots, kUnits);
    };
    auto variant = [&](const char *name, auto kernel, uint32_t blocks, uint32_t threads, size_t lds,
                       uint32_t units_per_block) {
        report(name, timer.median_us(run_push, [&] { launch_units(kernel, blocks, threads, lds, units_per_block); }),
               gather_bytes);
    };
    variant("  store nt (as the library)", gather_policy<kStoreNt>, kUnits, 64, 0, 1);
    variant("  store plain", gather_policy<kStorePlain>, kUnits, 64, 0, 1);
    variant("  store sc0 sc1", gather_policy<kStoreSc0Sc1>, kUnits, 64, 0, 1);
    variant("  store sc1", gather_policy<kStoreSc1>, kUnits, 64, 0, 1);
    variant("  store sc0", gather_policy<kStoreSc0>, kUnits, 64, 0, 1);
    variant("  store sc0 sc1 nt", gather_policy<kStoreSc0Sc1Nt>, kUnits, 64, 0, 1);
    variant("  cached loads, store nt", gather_cached_loads, kUnits, 64, 0, 1);
    variant("  pipelined, 2048 persistent wavefronts", gather_pipelined, 2048, 64, 0, 1);
    variant("  pipelined, 16384 persistent wavefronts", gather_pipelined, 16384, 64, 0, 1);
    variant("  a wavefront that only stores (3 + 1)", gather_store_wave, (kUnits + 2) / 3, 256, 0, 3);
    variant("  16 of 32 wavefronts per CU (10 KiB LDS each)", gather_policy<kStoreNt>, kUnits, 64, 10 * 1024, 1);
    variant("  8 of 32 wavefronts per CU (20 KiB LDS each)", gather_policy<kStoreNt>, kUnits, 64, 20 * 1024, 1);
    variant("  4 of 32 wavefronts per CU (40 KiB LDS each)", gather_policy<kStoreNt>, kUnits, 64, 40 * 1024, 1);
    variant("  a token's 14 pieces on one XCD", gather_mapped<1>, kUnits, 64, 0, 1);
    variant("  each XCD a contiguous eighth of the tokens", gather_mapped<2>, kUnits, 64, 0, 1);
    variant("  16 KiB bursts from LDS, 256 workgroups", gather_bursts<1>, 256, 1024, 16 * 1024, 16);
    variant("  64 KiB bursts from LDS, 512 workgroups", gather_bursts<4>, 512, 1024, 64 * 1024, 64);

    // Variants of the push: the cache policy of its stores, and half a token per workgroup.
    std::printf("variants of the push (after a gather):\n");
    auto push_variant = [&](const char *name, auto kernel, uint32_t blocks, uint32_t threads) {
        if (blocks == 0 || blocks > 2 * kTokens) {
            std::fprintf(stderr, "refusing a grid of %u workgroups for %u tokens\n", blocks, kTokens);
            std::exit(2);
        }
        report(name, timer.median_us(run_gather, [&] {
                   hipLaunchKernelGGL(kernel, dim3(blocks), dim3(threads), 0, s, (const uint8_t *)x, dispatched,
                                      (const uint32_t *)d_slots, kTokens);
               }),
               push_bytes);
    };
    push_variant("  store plain", (push_policy<kStorePlain, false>), kTokens, 448);
    push_variant("  store nt", (push_policy<kStoreNt, false>), kTokens, 448);
    push_variant("  store sc0 sc1 nt", (push_policy<kStoreSc0Sc1Nt, false>), kTokens, 448);
    push_variant("  store sc0", (push_policy<kStoreSc0, false>), kTokens, 448);
    push_variant("  store sc1 (as the library)", (push_policy<kStoreSc1, false>), kTokens, 448);
    push_variant("  store sc0 sc1", (push_policy<kStoreSc0Sc1, false>), kTokens, 448);
    push_variant("  store sc1, half a token per workgroup", (push_policy<kStoreSc1, true>), 2 * kTokens, 256);
    push_variant("  store sc1, 256 persistent workgroups", push_persistent, 256, 448);
    push_variant("  store sc1, each XCD a contiguous eighth", push_xcd_ranges, kTokens, 448);
    report("  pulled by destination row (input read 8 times)",
           timer.median_us(run_gather, [&] {
               hipLaunchKernelGGL(pull_by_row, dim3(kRows), dim3(448), 0, s, (const uint8_t *)x, dispatched,
                                  (const uint32_t *)d_token_of_row, kRows);
           }),
           push_bytes);

    // The same two shapes at 1024 tokens (the Kimi-K2 mixed batch): the push is a single wave of
    // workgroups, so nothing overlaps its launch, its reads and its burst of writes.
    std::printf("at 1024 tokens, push and gather in turn:\n");
    constexpr uint32_t kFewTokens = 1024;
    auto few_push = [&] {
        hipLaunchKernelGGL((push_policy<kStoreSc1, false>), dim3(kFewTokens), dim3(448), 0, s, (const uint8_t *)x,
                           dispatched, (const uint32_t *)d_slots, kFewTokens);
    };
    auto few_gather = [&] {
        hipLaunchKernelGGL(gather_policy<kStoreNt>, dim3(kFewTokens * kPieces), dim3(64), 0, s, (const uint8_t *)y,
                           combined, (const uint32_t *)d_slots, kFewTokens * kPieces);
    };
    report("  push, 1024 tokens, store sc1", timer.median_us(few_gather, few_push),
           (double)kFewTokens * (kInRow + kTopk * kOutRow));
    report("  gather, 1024 tokens", timer.median_us(few_push, few_gather),
           (double)kFewTokens * (kTopk + 1) * kInRow);
    return 0;
}
