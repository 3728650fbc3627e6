// A caller of the C ABI that uses nothing but the HIP runtime: what a host
// program in C or C++ (or a Rust `extern "C"` block) does with the library.
//
//   selftest            one small step through the group calls and one through
//                       the split calls, checked on the host; exit code 0 = ok
//
// The check is the round trip of the reference's own test
// (tests/p2p_all_to_all/test_p2p_all_to_all.py:44-50,182-189,233-234): with
// weights that sum to one, combine(dequantise(dispatch(x))) must give x back
// within the quantiser's error; and the expert counts the receivers report must
// equal a histogram of the indices made on the host.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "a2a.h"

#define HIP_OK(call)                                                                          \
    do {                                                                                      \
        hipError_t e_ = (call);                                                               \
        if (e_ != hipSuccess) {                                                               \
            std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));            \
            return 2;                                                                         \
        }                                                                                     \
    } while (0)
#define A2A_OK_OR_FAIL(call)                                                                  \
    do {                                                                                      \
        int rc_ = (call);                                                                     \
        if (rc_ != 0) {                                                                       \
            std::fprintf(stderr, "%s failed (%d): %s\n", #call, rc_, a2a_last_error(ctx));    \
            return 3;                                                                         \
        }                                                                                     \
    } while (0)

namespace {

constexpr uint32_t N = 4, E = 16, K = 2, H = 256, Hs = H / 128, T = 48, Le = E / N;

uint16_t to_bf16(float f) {
    uint32_t b;
    std::memcpy(&b, &f, 4);
    b += 0x7FFF + ((b >> 16) & 1);   // round to nearest even (finite inputs only)
    return (uint16_t)(b >> 16);
}

float from_bf16(uint16_t v) {
    uint32_t b = (uint32_t)v << 16;
    float f;
    std::memcpy(&f, &b, 4);
    return f;
}

float from_e4m3(uint8_t c) {   // OCP e4m3fn: bias 7, no infinities
    const int exp = (c >> 3) & 0xF, man = c & 7;
    const float mag = exp == 0 ? std::ldexp((float)man, -9) : std::ldexp(1.0f + man / 8.0f, exp - 7);
    return (c & 0x80) ? -mag : mag;
}

struct Rank {
    std::vector<uint16_t> x;         // [T][H] bf16
    std::vector<int32_t> idx;        // [T][K]
    std::vector<float> w;            // [T][K]
    void *d_x = nullptr, *d_idx = nullptr, *d_w = nullptr;
    void *d_n = nullptr, *d_ox = nullptr, *d_os = nullptr, *d_y = nullptr, *d_out = nullptr;
};

}  // namespace

int main() {
    int devices = 0;
    HIP_OK(hipGetDeviceCount(&devices));
    if (devices == 0) {
        std::fprintf(stderr, "no GPU\n");
        return 2;
    }
    HIP_OK(hipSetDevice(0));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));

    a2a_config cfg;
    std::memset(&cfg, 0, sizeof cfg);
    cfg.struct_size = sizeof cfg;
    cfg.hidden_dim = H;
    cfg.hidden_dim_scale = Hs;
    cfg.in_elemsize = 1;
    cfg.out_elemsize = 2;
    cfg.out_dtype = A2A_BF16;
    cfg.scale_elemsize = 4;
    cfg.max_num_tokens = T;
    cfg.max_recv_tokens = T * K * N;
    cfg.num_experts = E;
    cfg.expert_padding = 1;
    cfg.num_experts_per_token = K;
    cfg.dp_size = 1;
    cfg.node_size = N;
    cfg.world_size = N;
    cfg.device = 0;
    a2a_ctx *ctx = nullptr;
    A2A_OK_OR_FAIL(a2a_ctx_create(&cfg, &ctx));

    const size_t rows = (size_t)T * K * N;   // every copy could land on one rank
    std::vector<Rank> ranks(N);
    uint32_t seed = 12345;
    auto rnd = [&seed]() {
        seed = seed * 1664525u + 1013904223u;
        return (seed >> 8) * (1.0f / 16777216.0f);
    };
    std::vector<uint32_t> want_count(E, 0);
    for (uint32_t r = 0; r < N; ++r) {
        Rank &k = ranks[r];
        k.x.resize((size_t)T * H);
        k.idx.resize((size_t)T * K);
        k.w.assign((size_t)T * K, 1.0f / K);
        for (auto &v : k.x) v = to_bf16((rnd() - 0.5f) * 8.0f);
        for (uint32_t t = 0; t < T; ++t) {
            const uint32_t first = (uint32_t)(rnd() * E) % E;
            for (uint32_t j = 0; j < K; ++j) {   // K distinct experts
                k.idx[t * K + j] = (int32_t)((first + j * 5) % E);
                ++want_count[(first + j * 5) % E];
            }
        }
        HIP_OK(hipMalloc(&k.d_x, k.x.size() * 2));
        HIP_OK(hipMalloc(&k.d_idx, k.idx.size() * 4));
        HIP_OK(hipMalloc(&k.d_w, k.w.size() * 4));
        HIP_OK(hipMalloc(&k.d_n, Le * 4));
        HIP_OK(hipMalloc(&k.d_ox, rows * H));
        HIP_OK(hipMalloc(&k.d_os, rows * Hs * 4));
        HIP_OK(hipMalloc(&k.d_y, rows * H * 2));
        HIP_OK(hipMalloc(&k.d_out, (size_t)T * H * 2));
        HIP_OK(hipMemcpy(k.d_x, k.x.data(), k.x.size() * 2, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(k.d_idx, k.idx.data(), k.idx.size() * 4, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(k.d_w, k.w.data(), k.w.size() * 4, hipMemcpyHostToDevice));
    }

    int failures = 0;
    for (int split = 0; split < 2; ++split) {
        for (Rank &k : ranks) {
            HIP_OK(hipMemset(k.d_ox, 0, rows * H));
            HIP_OK(hipMemset(k.d_os, 0, rows * Hs * 4));
            HIP_OK(hipMemset(k.d_out, 0, (size_t)T * H * 2));
        }
        if (!split) {
            a2a_dispatch_args d[N];
            std::memset(d, 0, sizeof d);
            for (uint32_t r = 0; r < N; ++r) {
                Rank &k = ranks[r];
                d[r].num_tokens = T;
                d[r].x_ptr = k.d_x;
                d[r].x_stride = H * 2;
                d[r].indices = (const int32_t *)k.d_idx;
                d[r].indices_stride = K;
                d[r].weights = (const float *)k.d_w;
                d[r].weights_stride = K;
                d[r].out_num_tokens = (int32_t *)k.d_n;
                d[r].out_x = k.d_ox;
                d[r].out_x_stride = H;
                d[r].out_x_rows = rows;
                d[r].out_x_scale = (float *)k.d_os;
                d[r].out_x_scale_stride_elem = 1;
                d[r].out_x_scale_stride_token = Hs;
            }
            A2A_OK_OR_FAIL(a2a_dispatch(ctx, d, /*quantize=*/1, stream));
        } else {
            for (uint32_t r = 0; r < N; ++r) {
                Rank &k = ranks[r];
                A2A_OK_OR_FAIL(a2a_dispatch_send(ctx, r, T, k.d_x, H * 2, 1, nullptr, 0, 0, (const int32_t *)k.d_idx, K,
                                                 (const float *)k.d_w, K, nullptr, stream));
            }
            for (uint32_t r = 0; r < N; ++r) {
                Rank &k = ranks[r];
                A2A_OK_OR_FAIL(a2a_dispatch_recv(ctx, r, (int32_t *)k.d_n, k.d_ox, H, rows, (float *)k.d_os, 1, Hs,
                                                 stream));
            }
        }
        HIP_OK(hipStreamSynchronize(stream));

        // expert counts, and the experts' stand-in: y = dequantised row, as bf16
        for (uint32_t r = 0; r < N; ++r) {
            Rank &k = ranks[r];
            int32_t n[Le];
            HIP_OK(hipMemcpy(n, k.d_n, sizeof n, hipMemcpyDeviceToHost));
            for (uint32_t le = 0; le < Le; ++le) {
                if ((uint32_t)n[le] != want_count[r * Le + le]) {
                    std::fprintf(stderr, "split=%d rank %u expert %u: %d rows, expected %u\n", split, r, le, n[le],
                                 want_count[r * Le + le]);
                    ++failures;
                }
            }
            std::vector<uint8_t> q(rows * H);
            std::vector<float> s(rows * Hs);
            std::vector<uint16_t> y(rows * H);
            HIP_OK(hipMemcpy(q.data(), k.d_ox, q.size(), hipMemcpyDeviceToHost));
            HIP_OK(hipMemcpy(s.data(), k.d_os, s.size() * 4, hipMemcpyDeviceToHost));
            for (size_t row = 0; row < rows; ++row) {
                for (uint32_t h = 0; h < H; ++h) {
                    y[row * H + h] = to_bf16(from_e4m3(q[row * H + h]) * s[row * Hs + h / 128]);
                }
            }
            HIP_OK(hipMemcpy(k.d_y, y.data(), y.size() * 2, hipMemcpyHostToDevice));
        }

        if (!split) {
            a2a_combine_args c[N];
            std::memset(c, 0, sizeof c);
            for (uint32_t r = 0; r < N; ++r) {
                Rank &k = ranks[r];
                c[r].expert_y = k.d_y;
                c[r].expert_y_stride = H * 2;
                c[r].expert_y_rows = rows;
                c[r].num_tokens = T;
                c[r].out_tokens = k.d_out;
                c[r].out_tokens_stride = H;
                c[r].indices = (const int32_t *)k.d_idx;
                c[r].indices_stride = K;
                c[r].weights = (const float *)k.d_w;
                c[r].weights_stride = K;
            }
            A2A_OK_OR_FAIL(a2a_combine(ctx, c, A2A_BF16, /*accumulate=*/0, stream));
        } else {
            for (uint32_t r = 0; r < N; ++r) {
                A2A_OK_OR_FAIL(a2a_combine_send(ctx, r, ranks[r].d_y, H * 2, rows, stream));
            }
            for (uint32_t r = 0; r < N; ++r) {
                Rank &k = ranks[r];
                A2A_OK_OR_FAIL(a2a_combine_recv(ctx, r, T, 0, A2A_BF16, k.d_out, H, (const int32_t *)k.d_idx, K,
                                                (const float *)k.d_w, K, nullptr, 0, stream));
            }
        }
        uint32_t flags = 0;
        A2A_OK_OR_FAIL(a2a_ctx_status(ctx, stream, &flags));
        if (flags != 0) {
            std::fprintf(stderr, "split=%d: device error flags 0x%x\n", split, flags);
            ++failures;
        }

        // every copy of a token is the same quantised row, so the mean of K copies is that row:
        // within one fp8 step of the input (2^-3 relative) plus bf16 rounding
        double worst = 0.0;
        for (uint32_t r = 0; r < N; ++r) {
            Rank &k = ranks[r];
            std::vector<uint16_t> out((size_t)T * H);
            HIP_OK(hipMemcpy(out.data(), k.d_out, out.size() * 2, hipMemcpyDeviceToHost));
            for (size_t i = 0; i < out.size(); ++i) {
                const float want = from_bf16(k.x[i]), got = from_bf16(out[i]);
                const double err = std::fabs(got - want) / (std::fabs(want) + 0.25);
                if (err > worst) worst = err;
            }
        }
        std::printf("%s calls: expert counts ok, round trip within %.3f of the input\n", split ? "split" : "group",
                    worst);
        if (worst > 0.08) {
            std::fprintf(stderr, "split=%d: round trip error %.3f\n", split, worst);
            ++failures;
        }
    }

    // a2a_dispatch_static: no context, no allocation; must write what a2a_dispatch writes.
    {
        a2a_dispatch_args d[N], d2[N];
        std::memset(d, 0, sizeof d);
        std::vector<void *> n2(N), ox2(N), os2(N);
        uint32_t *d_flags = nullptr;
        HIP_OK(hipMalloc(&d_flags, sizeof(uint32_t)));
        HIP_OK(hipMemset(d_flags, 0, sizeof(uint32_t)));
        for (uint32_t r = 0; r < N; ++r) {
            Rank &k = ranks[r];
            HIP_OK(hipMalloc(&n2[r], Le * 4));
            HIP_OK(hipMalloc(&ox2[r], rows * H));
            HIP_OK(hipMalloc(&os2[r], rows * Hs * 4));
            HIP_OK(hipMemset(k.d_ox, 0, rows * H));
            HIP_OK(hipMemset(k.d_os, 0, rows * Hs * 4));
            HIP_OK(hipMemset(ox2[r], 0, rows * H));
            HIP_OK(hipMemset(os2[r], 0, rows * Hs * 4));
            d[r].num_tokens = T;
            d[r].x_ptr = k.d_x;
            d[r].x_stride = H * 2;
            d[r].indices = (const int32_t *)k.d_idx;
            d[r].indices_stride = K;
            d[r].out_num_tokens = (int32_t *)k.d_n;
            d[r].out_x = k.d_ox;
            d[r].out_x_stride = H;
            d[r].out_x_rows = rows;
            d[r].out_x_scale = (float *)k.d_os;
            d[r].out_x_scale_stride_elem = 1;
            d[r].out_x_scale_stride_token = Hs;
            d2[r] = d[r];
            d2[r].out_num_tokens = (int32_t *)n2[r];
            d2[r].out_x = ox2[r];
            d2[r].out_x_scale = (float *)os2[r];
        }
        // The FIRST call on a GPU looks up the library's array there, which a stream capture forbids:
        // it is refused, and the refusal leaves nothing in the graph.
        auto captured = [&](const a2a_dispatch_args *args, int *rc_out, size_t *nodes_out) -> int {
            hipGraph_t graph = nullptr;
            HIP_OK(hipStreamBeginCapture(stream, hipStreamCaptureModeRelaxed));
            *rc_out = a2a_dispatch_static(&cfg, args, /*quantize=*/1, d_flags, stream);
            HIP_OK(hipStreamEndCapture(stream, &graph));
            *nodes_out = 99;
            HIP_OK(hipGraphGetNodes(graph, nullptr, nodes_out));
            HIP_OK(hipGraphDestroy(graph));
            return 0;
        };
        int rc_cap = 0;
        size_t nodes = 0;
        if (int e = captured(d2, &rc_cap, &nodes)) return e;
        const bool first_refused = rc_cap == A2A_ERR_BAD_ORDER && nodes == 0;
        std::printf("static dispatch, first call under capture: %s (%d, %zu nodes)\n",
                    first_refused ? "refused" : "NOT REFUSED", rc_cap, nodes);
        if (!first_refused) ++failures;

        A2A_OK_OR_FAIL(a2a_dispatch(ctx, d, /*quantize=*/1, stream));
        const int rc = a2a_dispatch_static(&cfg, d2, /*quantize=*/1, d_flags, stream);
        if (rc != 0) {
            std::fprintf(stderr, "a2a_dispatch_static failed (%d): %s\n", rc, a2a_last_error(nullptr));
            return 1;
        }
        HIP_OK(hipStreamSynchronize(stream));
        uint32_t flags = 1;
        HIP_OK(hipMemcpy(&flags, d_flags, sizeof flags, hipMemcpyDeviceToHost));
        bool same = flags == 0;
        std::vector<uint8_t> a(rows * H), b(rows * H);
        std::vector<float> sa(rows * Hs), sb(rows * Hs);
        for (uint32_t r = 0; r < N && same; ++r) {
            int32_t na[Le], nb[Le];
            HIP_OK(hipMemcpy(na, ranks[r].d_n, sizeof na, hipMemcpyDeviceToHost));
            HIP_OK(hipMemcpy(nb, n2[r], sizeof nb, hipMemcpyDeviceToHost));
            HIP_OK(hipMemcpy(a.data(), ranks[r].d_ox, a.size(), hipMemcpyDeviceToHost));
            HIP_OK(hipMemcpy(b.data(), ox2[r], b.size(), hipMemcpyDeviceToHost));
            HIP_OK(hipMemcpy(sa.data(), ranks[r].d_os, sa.size() * 4, hipMemcpyDeviceToHost));
            HIP_OK(hipMemcpy(sb.data(), os2[r], sb.size() * 4, hipMemcpyDeviceToHost));
            same = std::memcmp(na, nb, sizeof na) == 0 && a == b &&
                   std::memcmp(sa.data(), sb.data(), sa.size() * 4) == 0;
        }
        std::printf("static dispatch: %s\n", same ? "identical to a2a_dispatch" : "DIFFERS from a2a_dispatch");
        if (!same) ++failures;
        // After that eager call a capture takes the launches; a call that is refused (tokens without
        // rows) still records none: every check runs before the first launch.
        a2a_dispatch_args bad[N];
        std::memcpy(bad, d2, sizeof bad);
        bad[N - 1].x_ptr = nullptr;
        if (int e = captured(bad, &rc_cap, &nodes)) return e;
        const bool clean_refusal = rc_cap == A2A_ERR_INVALID_ARGUMENT && nodes == 0;
        if (int e = captured(d2, &rc_cap, &nodes)) return e;
        const bool recorded = rc_cap == 0 && nodes >= 2;
        std::printf("static dispatch under capture: refused call %s, accepted call %s (%zu nodes)\n",
                    clean_refusal ? "recorded nothing" : "LEFT NODES BEHIND", recorded ? "recorded" : "NOT RECORDED",
                    nodes);
        if (!clean_refusal || !recorded) ++failures;
        for (uint32_t r = 0; r < N; ++r) {
            (void)hipFree(n2[r]);
            (void)hipFree(ox2[r]);
            (void)hipFree(os2[r]);
        }
        (void)hipFree(d_flags);
    }

    for (Rank &k : ranks) {
        for (void *p : {k.d_x, k.d_idx, k.d_w, k.d_n, k.d_ox, k.d_os, k.d_y, k.d_out}) (void)hipFree(p);
    }
    A2A_OK_OR_FAIL(a2a_ctx_destroy(ctx));
    (void)hipStreamDestroy(stream);
    std::printf(failures == 0 ? "selftest passed\n" : "selftest FAILED\n");
    return failures == 0 ? 0 : 1;
}
