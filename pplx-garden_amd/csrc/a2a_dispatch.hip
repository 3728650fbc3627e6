// Dispatch pack: read every token row once, optionally quantise it to fp8 e4m3
// with one float scale per 128 elements, and write one copy per route straight
// into the receiver's rows.
//
// What it replaces: phase 2 of the reference's dispatch-send kernel (row ->
// staging buffer per route, a2a_dispatch_send.cu:266-523) fused with the
// dispatch-recv kernel (staging -> out_x[padded_index], a2a_dispatch_recv.cu:
// 122-156).  The reference moves every copy twice; here it moves once.
//
// Design for CDNA4: one workgroup per token, one 16-byte fp8 store per lane per
// route.  In quantise mode a lane owns 16 consecutive bf16 (two 16-byte loads),
// so a 128-element scale group is exactly 8 lanes, i.e. half a DPP row: the
// group maximum takes two quad permutes and one half-row mirror, no LDS.  The
// eight scales a wavefront produces are spread over the lanes so that a single
// store instruction writes them for eight routes at once.  Row pointers are
// computed once per token by the first K lanes and read back as wave-uniform
// scalars.  Token rows are loaded non-temporally (each is read once).  The
// copies are written with ordinary stores: measured on this part, non-temporal
// stores to this many rows at once sustain about two thirds of that rate, and
// what ordinary stores leave in the cache is what the experts read next.
#include "a2a_device.h"

namespace a2a {

template <bool QUANT>
__global__ __launch_bounds__(1024) void dispatch_push_kernel(const PushArgs args,
                                                             const Workspace ws) {
    // Scales of one token (one per 128 elements) and where each copy's go.
    constexpr int kMaxLdsScales = 1024;
    __shared__ float s_scale[QUANT ? kMaxLdsScales : 1];
    __shared__ uint64_t s_scale_ptr[A2A_MAX_EXPERTS_PER_TOKEN];
    __shared__ uint32_t s_scale_stride[A2A_MAX_EXPERTS_PER_TOKEN];

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const uint32_t E = ws.num_experts;
    const uint32_t K = ws.topk;

    uint32_t g = 0;
    while (g + 1 < ws.num_groups && blockIdx.x >= args.token_start[g + 1]) ++g;
    const uint32_t token = blockIdx.x - args.token_start[g];
    const PushSrc &src = args.src[g];
    if (token >= effective_tokens(src.bound_m, src.num_tokens)) return;

    // Lanes 0..K-1 of every wavefront resolve one route each.
    uint64_t row_ptr = 0, scale_ptr = 0;
    uint32_t scale_stride = 0;
    if (lane < K) {
        const uint32_t entry = token * K + lane;
        const uint32_t expert =
            (uint32_t)src.indices[(size_t)token * src.indices_stride + lane];
        uint32_t slot = kInvalidSlot, toff = 0;
        if (expert < E) {
            const uint32_t chunk = entry / kRouteBlock;
            toff = ws.block_prefix[((size_t)g * ws.nb_max + chunk) * E + expert] +
                   ws.local_rank[(size_t)g * ws.max_tk + entry];
            slot = ws.slot_base[g * E + expert] + toff;
            const PushDst &dst = args.dst[expert / ws.experts_per_rank];
            if (dst.out_x != nullptr) {
                if (slot < dst.out_rows) {
                    row_ptr = (uint64_t)(dst.out_x + (size_t)slot * dst.out_stride);
                    if (dst.out_scale != nullptr) {
                        scale_ptr = (uint64_t)(dst.out_scale + (size_t)slot * dst.os_stride_token);
                        scale_stride = dst.os_stride_elem;
                    }
                } else {
                    slot = kInvalidSlot;
                    if (wave == 0) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
                }
            }
        }
        if (wave == 0) {
            ws.route_slot[(size_t)g * ws.max_tk + entry] = slot;
            ws.token_offset[(size_t)g * ws.max_tk + entry] = toff;
        }
    }

    const uint8_t *x_row = src.x + (size_t)token * src.x_stride;

    if constexpr (QUANT) {
        const uint32_t num_chunks = args.hidden_dim / 16;  // 16 bf16 in, 16 fp8 out per lane
        const uint32_t Hs = args.hidden_dim_scale;
        for (uint32_t base = wave * kWave; base < num_chunks; base += blockDim.x) {
            const uint32_t c = base + lane;
            const bool active = c < num_chunks;
            u32x4 a = {0, 0, 0, 0}, b = {0, 0, 0, 0};
            if (active) {
                const u32x4 *p = reinterpret_cast<const u32x4 *>(x_row + (size_t)c * 32);
                a = __builtin_nontemporal_load(p);
                b = __builtin_nontemporal_load(p + 1);
            }
            float scale;
            const u32x4 q = quantize16(a, b, &scale);
            for (uint32_t k = 0; k < K; ++k) {
                const uint64_t row = read_lane64(row_ptr, k);
                if (row != 0 && active) {
                    *reinterpret_cast<u32x4 *>(row + (size_t)c * 16) = q;
                }
            }
            if (active && (lane & 7) == 0 && c / 8 < kMaxLdsScales) s_scale[c / 8] = scale;
        }
        // The token's scales meet in LDS so that each copy's scale row goes out
        // as one contiguous run instead of one 32-byte piece per wavefront.
        if (wave == 0 && lane < K) {
            s_scale_ptr[lane] = scale_ptr;
            s_scale_stride[lane] = scale_stride;
        }
        __syncthreads();
        const uint32_t Hl = Hs < (uint32_t)kMaxLdsScales ? Hs : (uint32_t)kMaxLdsScales;
        for (uint32_t i = tid; i < K * Hl; i += blockDim.x) {
            const uint32_t k = i / Hl;
            const uint32_t j = i - k * Hl;
            const uint64_t sp = s_scale_ptr[k];
            if (sp != 0) reinterpret_cast<float *>(sp)[(size_t)j * s_scale_stride[k]] = s_scale[j];
        }
    } else {
        const uint32_t num_chunks = args.row_bytes / 16;
        for (uint32_t c = tid; c < num_chunks; c += blockDim.x) {
            const u32x4 v =
                __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x_row) + c);
            for (uint32_t k = 0; k < K; ++k) {
                const uint64_t row = read_lane64(row_ptr, k);
                if (row != 0) {
                    reinterpret_cast<u32x4 *>(row)[c] = v;
                }
            }
        }
        if (src.x_scale != nullptr) {
            const float *xs = src.x_scale + (size_t)token * src.xs_stride_token;
            for (uint32_t j = tid; j < args.hidden_dim_scale; j += blockDim.x) {
                const float s = xs[(size_t)j * src.xs_stride_elem];
                for (uint32_t k = 0; k < K; ++k) {
                    const uint64_t sp = read_lane64(scale_ptr, k);
                    const uint32_t ss = __builtin_amdgcn_readlane((int)scale_stride, (int)k);
                    if (sp != 0) reinterpret_cast<float *>(sp)[(size_t)j * ss] = s;
                }
            }
        }
    }
}

hipError_t launch_dispatch_push(const PushArgs &args, const Workspace &ws, bool quantize,
                                uint32_t total_tokens, hipStream_t stream) {
    if (total_tokens == 0) return hipSuccess;
    const uint32_t chunks = quantize ? args.hidden_dim / 16 : args.row_bytes / 16;
#ifndef A2A_PUSH_SLABS
#define A2A_PUSH_SLABS 1
#endif
    uint32_t threads = ((chunks + kWave - 1) / kWave + A2A_PUSH_SLABS - 1) / A2A_PUSH_SLABS * kWave;
    if (threads < (uint32_t)kWave) threads = kWave;
    if (threads > 1024) threads = 1024;
    if (quantize) {
        hipLaunchKernelGGL(dispatch_push_kernel<true>, dim3(total_tokens), dim3(threads), 0, stream,
                           args, ws);
    } else {
        hipLaunchKernelGGL(dispatch_push_kernel<false>, dim3(total_tokens), dim3(threads), 0,
                           stream, args, ws);
    }
    return hipGetLastError();
}

}  // namespace a2a
