// Kernels of the split calls; see a2a_staged.h for what they mirror.
#include "a2a_staged.h"

#include <cstring>

#include "a2a_device.h"

namespace a2a {

namespace {

size_t align_up_sz(size_t n, size_t a) { return (n + a - 1) / a * a; }

// ---------------------------------------------------------------------------
// dispatch send: stage one (quantised) row per token, record which token sits
// behind every row of the sender's expert-sorted order.
// ---------------------------------------------------------------------------
template <bool QUANT>
__global__ __launch_bounds__(1024) void stage_send_kernel(const StageSendArgs args, const Workspace ws,
                                                          const Staging st) {
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t wave = tid / kWave;
    const uint32_t E = ws.num_experts;
    const uint32_t K = ws.topk;
    const uint32_t g = args.rank / ws.dp_size;   // ranks of a dp group hold the same tokens
    const uint32_t token = blockIdx.x;
    const PushSrc &src = args.src;
    if (token >= effective_tokens(src.bound_m, src.num_tokens)) return;

    if (wave == 0 && lane < K) {
        const uint32_t entry = token * K + lane;
        const uint32_t expert = (uint32_t)src.indices[(size_t)token * src.indices_stride + lane];
        uint32_t toff = 0;
        if (expert < E) {
            toff = ws.block_prefix[((size_t)g * ws.nb_max + entry / kRouteBlock) * E + expert] +
                   ws.local_rank[(size_t)g * ws.max_tk + entry];
            // position of the copy (a2a_dispatch_send.cu:54)
            const uint32_t excl = expert > 0 ? ws.expert_offsets[g * E + expert - 1] : 0;
            st.pos_token[(size_t)g * ws.max_tk + excl + toff] = token;
        }
        ws.token_offset[(size_t)g * ws.max_tk + entry] = toff;
    }

    const uint8_t *x_row = src.x + (size_t)token * src.x_stride;
    uint8_t *row = st.send_buf + ((size_t)g * st.max_tokens + token) * st.disp_stride;
    float *row_scale = reinterpret_cast<float *>(row + st.payload_bytes);

    if constexpr (QUANT) {
        const uint32_t num_chunks = args.hidden_dim / 16;
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
            if (active) {
                reinterpret_cast<u32x4 *>(row)[c] = q;
                if ((lane & 7) == 0) row_scale[c / 8] = scale;
            }
        }
    } else {
        const uint32_t num_chunks = args.row_bytes / 16;
        for (uint32_t c = tid; c < num_chunks; c += blockDim.x) {
            reinterpret_cast<u32x4 *>(row)[c] =
                __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x_row) + c);
        }
        if (src.x_scale != nullptr) {
            const float *xs = src.x_scale + (size_t)token * src.xs_stride_token;
            for (uint32_t j = tid; j < args.hidden_dim_scale; j += blockDim.x) {
                row_scale[j] = xs[(size_t)j * src.xs_stride_elem];
            }
        }
    }
}

// ---------------------------------------------------------------------------
// dispatch recv, step 1: first received row of every (source, local expert)
// run, in the order the reference's host worker visits them
// (a2a_worker.rs:621-634,681-694).  One workgroup.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void recv_segments_kernel(const StageRecvArgs args,
                                                             const Workspace ws, const Staging st) {
    __shared__ uint32_t wave_tot[16];
    __shared__ uint32_t carry_s;
    const uint32_t G = ws.num_groups, E = ws.num_experts, Le = ws.experts_per_rank;
    const uint32_t r = args.rank;
    const uint32_t first = r * Le;
    const uint32_t n_local = first >= E ? 0 : (E - first < Le ? E - first : Le);
    const uint32_t num_seg = G * Le;
    uint32_t *seg = st.seg_start + (size_t)r * (ws.world * Le + 1);
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t remote_segs = (ws.world / ws.node_size - 1) * (ws.node_size / ws.dp_size) * Le;

    if (tid == 0) carry_s = 0;
    __syncthreads();
    for (uint32_t base = 0; base < num_seg; base += blockDim.x) {
        const uint32_t s = base + tid;
        uint32_t cnt = 0;
        if (s < num_seg) {
            const uint32_t g = source_order_lookup(ws.order, r, s / Le);
            const uint32_t le = s % Le;
            if (le < n_local && (args.valid_mask >> g & 1)) cnt = ws.num_routed[g * E + first + le];
        }
        // block-wide exclusive scan of cnt
        uint32_t incl = cnt;
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1) {
            const uint32_t up = __shfl_up(incl, d);
            if (lane >= (uint32_t)d) incl += up;
        }
        if (lane == kWave - 1) wave_tot[wave] = incl;
        __syncthreads();
        uint32_t before = carry_s;
        for (uint32_t w = 0; w < wave; ++w) before += wave_tot[w];
        if (s < num_seg) seg[s] = before + incl - cnt;
        __syncthreads();
        if (tid == blockDim.x - 1) carry_s = before + incl;
        __syncthreads();
    }
    if (tid == 0) {
        const uint32_t total = carry_s;
        seg[num_seg] = total;
        st.num_recv[2 * r] = total;
        // rows that come from other nodes (num_efa_tokens, a2a_worker.rs:681-687)
        st.num_recv[2 * r + 1] = remote_segs < num_seg ? seg[remote_segs] : total;
    }
}

// Locate received row `i` of receiver `r`: its run (source, local expert) and
// its index inside the run.  Binary search over seg_start (ascending).
__device__ __forceinline__ void locate_row(const uint32_t *seg, uint32_t num_seg, uint32_t i,
                                           uint32_t *seg_out, uint32_t *j_out) {
    uint32_t lo = 0, hi = num_seg;  // seg[lo] <= i < seg[hi]
    while (hi - lo > 1) {
        const uint32_t mid = (lo + hi) / 2;
        if (seg[mid] <= i) lo = mid; else hi = mid;
    }
    *seg_out = lo;
    *j_out = i - seg[lo];
}

// ---------------------------------------------------------------------------
// dispatch recv, step 2: one workgroup per received row.  Writes the row's
// metadata (padded_index, source_rank, source position: a2a_worker.rs:636-671)
// and copies payload and scales from the sender's staged token
// (a2a_dispatch_recv.cu:139-155).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void stage_recv_kernel(const StageRecvArgs args, const Workspace ws,
                                                          const Staging st) {
    const uint32_t E = ws.num_experts, Le = ws.experts_per_rank;
    const uint32_t r = args.rank;
    const uint32_t num_seg = ws.num_groups * Le;
    const uint32_t *seg = st.seg_start + (size_t)r * (ws.world * Le + 1);
    const uint32_t i = blockIdx.x;
    if (i >= seg[num_seg]) return;
    uint32_t s, j;
    locate_row(seg, num_seg, i, &s, &j);
    const uint32_t g = source_order_lookup(ws.order, r, s / Le);
    const uint32_t e = r * Le + s % Le;
    const uint32_t excl = e > 0 ? ws.expert_offsets[g * E + e - 1] : 0;
    const uint32_t pos = excl + j;
    const uint32_t dst_row = ws.slot_base[g * E + e] + j;
    const uint32_t tid = threadIdx.x;
    if (tid == 0 && i < st.max_recv) {
        st.padded_index[(size_t)r * st.max_recv + i] = dst_row;
        // the member of the group that sends to this rank (a2a_worker.rs:633)
        st.source_rank[(size_t)r * st.max_recv + i] = g * ws.dp_size + r % ws.dp_size;
        st.source_position[(size_t)r * st.max_recv + i] = pos;
    }
    const PushDst &dst = args.dst;
    if (dst.out_x == nullptr) return;
    if (dst_row >= dst.out_rows) {
        if (tid == 0) atomicOr(ws.err, A2A_DEV_RECV_OVERFLOW);
        return;
    }
    const uint32_t token = st.pos_token[(size_t)g * ws.max_tk + pos];
    const uint8_t *src = st.send_buf + ((size_t)g * st.max_tokens + token) * st.disp_stride;
    uint8_t *out = dst.out_x + (size_t)dst_row * dst.out_stride;
    const uint32_t num_chunks = args.row_bytes / 16;
    for (uint32_t c = tid; c < num_chunks; c += blockDim.x) {
        __builtin_nontemporal_store(reinterpret_cast<const u32x4 *>(src)[c],
                                    reinterpret_cast<u32x4 *>(out) + c);
    }
    if (dst.out_scale != nullptr) {
        const float *ss = reinterpret_cast<const float *>(src + st.payload_bytes);
        float *os = dst.out_scale + (size_t)dst_row * dst.os_stride_token;
        for (uint32_t q = tid; q < args.hidden_dim_scale; q += blockDim.x) {
            os[(size_t)q * dst.os_stride_elem] = ss[q];
        }
    }
}

// ---------------------------------------------------------------------------
// combine send: copy expert_y[padded_index[i]] to the staging row of the copy
// it answers, i.e. row `source_position[i]` of sender `source_rank[i]`
// (a2a_combine_send.cu:124-136,196-205).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void combine_send_kernel(const CombineSendArgs args,
                                                            const Workspace ws, const Staging st) {
    const uint32_t r = args.rank;
    const uint32_t i = blockIdx.x;
    if (i >= st.num_recv[2 * r] || i >= st.max_recv) return;
    const uint32_t row = st.padded_index[(size_t)r * st.max_recv + i];
    // every member of the source's dp group reads the same staging rows
    const uint32_t g = st.source_rank[(size_t)r * st.max_recv + i] / ws.dp_size;
    const uint32_t pos = st.source_position[(size_t)r * st.max_recv + i];
    if (row >= args.y_rows || pos >= ws.max_tk) {
        if (threadIdx.x == 0) atomicOr(ws.err, A2A_DEV_BAD_SLOT);
        return;
    }
    const u32x4 *src = reinterpret_cast<const u32x4 *>(args.y + (size_t)row * args.y_stride);
    u32x4 *dst = reinterpret_cast<u32x4 *>(st.comb_buf + ((size_t)g * ws.max_tk + pos) * st.comb_stride);
    const uint32_t num_chunks = args.row_bytes / 16;
    for (uint32_t c = threadIdx.x; c < num_chunks; c += blockDim.x) {
        dst[c] = __builtin_nontemporal_load(src + c);
    }
}

uint32_t block_for_chunks(uint32_t chunks) {
    uint32_t threads = (chunks + kWave - 1) / kWave * kWave;
    if (threads < (uint32_t)kWave) threads = kWave;
    if (threads > 1024) threads = 1024;
    return threads;
}

}  // namespace

int staging_allocate(Staging &st, const a2a_config &cfg, std::string *error) {
    if (st.allocated) return A2A_OK;
    const size_t N = cfg.world_size;
    const size_t K = cfg.num_experts_per_token;
    const size_t max_tk = (size_t)cfg.max_num_tokens * K;
    const size_t Le = (cfg.num_experts + N - 1) / N;
    st.disp_stride = a2a_dispatch_token_stride(&cfg);
    st.comb_stride = a2a_combine_token_stride(&cfg);
    st.payload_bytes = (uint32_t)align_up_sz((size_t)cfg.hidden_dim * cfg.in_elemsize, 16);
    st.max_tokens = cfg.max_num_tokens;
    // A receiver can get every copy of every sender.
    const size_t max_recv = N * max_tk;
    if (max_recv > 0x7FFFFFFFull) {
        if (error) *error = "world_size * max_num_tokens * num_experts_per_token too large";
        return A2A_ERR_UNSUPPORTED;
    }
    st.max_recv = (uint32_t)max_recv;

    size_t off = 0;
    auto carve = [&off](size_t bytes) {
        const size_t at = off;
        off = align_up_sz(off + bytes, 256);
        return at;
    };
    const size_t o_send = carve(N * cfg.max_num_tokens * st.disp_stride);
    const size_t o_pos = carve(N * max_tk * sizeof(uint32_t));
    const size_t o_comb = carve(N * max_tk * st.comb_stride);
    const size_t o_seg = carve(N * (N * Le + 1) * sizeof(uint32_t));
    const size_t o_pidx = carve(N * max_recv * sizeof(uint32_t));
    const size_t o_srank = carve(N * max_recv * sizeof(uint32_t));
    const size_t o_spos = carve(N * max_recv * sizeof(uint32_t));
    const size_t o_nrecv = carve(N * 2 * sizeof(uint32_t));
    hipError_t e = hipMalloc(&st.arena, off);
    if (e != hipSuccess) {
        if (error) {
            *error = "hipMalloc(staging, " + std::to_string(off) + " bytes): " + hipGetErrorString(e);
        }
        st.arena = nullptr;
        return A2A_ERR_OUT_OF_MEMORY;
    }
    uint8_t *base = static_cast<uint8_t *>(st.arena);
    st.send_buf = base + o_send;
    st.pos_token = reinterpret_cast<uint32_t *>(base + o_pos);
    st.comb_buf = base + o_comb;
    st.seg_start = reinterpret_cast<uint32_t *>(base + o_seg);
    st.padded_index = reinterpret_cast<uint32_t *>(base + o_pidx);
    st.source_rank = reinterpret_cast<uint32_t *>(base + o_srank);
    st.source_position = reinterpret_cast<uint32_t *>(base + o_spos);
    st.num_recv = reinterpret_cast<uint32_t *>(base + o_nrecv);
    // Tables are read before they are written only through misuse; start from zero.
    e = hipMemset(base + o_pos, 0, o_comb - o_pos);
    if (e == hipSuccess) e = hipMemset(base + o_seg, 0, off - o_seg);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) {
        if (error) *error = std::string("hipMemset(staging): ") + hipGetErrorString(e);
        (void)hipFree(st.arena);
        st.arena = nullptr;
        return (int)e;
    }
    st.allocated = true;
    return A2A_OK;
}

void staging_free(Staging &st) {
    if (st.arena != nullptr) (void)hipFree(st.arena);
    st = Staging();
}

const uint32_t *staging_table(const Staging &st, const a2a_config &cfg, uint32_t rank, uint32_t which,
                              size_t *limit) {
    (void)cfg;
    if (!st.allocated || !(st.recv_mask >> rank & 1)) return nullptr;
    switch (which) {
        case A2A_TABLE_PADDED_INDEX:
            *limit = st.max_recv;
            return st.padded_index + (size_t)rank * st.max_recv;
        case A2A_TABLE_SOURCE_RANK:
            *limit = st.max_recv;
            return st.source_rank + (size_t)rank * st.max_recv;
        case A2A_TABLE_SOURCE_POSITION:
            *limit = st.max_recv;
            return st.source_position + (size_t)rank * st.max_recv;
        case A2A_TABLE_NUM_RECV_TOKENS:
            *limit = 2;
            return st.num_recv + (size_t)rank * 2;
        default:
            return nullptr;
    }
}

hipError_t launch_stage_send(const StageSendArgs &args, const Workspace &ws, const Staging &st,
                             bool quantize, hipStream_t stream) {
    if (args.src.num_tokens == 0) return hipSuccess;
    const uint32_t threads = block_for_chunks(quantize ? args.hidden_dim / 16 : args.row_bytes / 16);
    if (quantize) {
        hipLaunchKernelGGL(stage_send_kernel<true>, dim3(args.src.num_tokens), dim3(threads), 0, stream,
                           args, ws, st);
    } else {
        hipLaunchKernelGGL(stage_send_kernel<false>, dim3(args.src.num_tokens), dim3(threads), 0, stream,
                           args, ws, st);
    }
    return hipGetLastError();
}

hipError_t launch_stage_recv(const StageRecvArgs &args, const Workspace &ws, const Staging &st,
                             hipStream_t stream) {
    uint32_t seg_threads = (ws.num_groups * ws.experts_per_rank + kWave - 1) / kWave * kWave;
    if (seg_threads > 1024) seg_threads = 1024;
    hipLaunchKernelGGL(recv_segments_kernel, dim3(1), dim3(seg_threads), 0, stream, args, ws, st);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || args.max_rows == 0) return e;
    hipLaunchKernelGGL(stage_recv_kernel, dim3(args.max_rows), dim3(block_for_chunks(args.row_bytes / 16)),
                       0, stream, args, ws, st);
    return hipGetLastError();
}

hipError_t launch_combine_send(const CombineSendArgs &args, const Workspace &ws, const Staging &st,
                               hipStream_t stream) {
    if (args.max_rows == 0) return hipSuccess;
    hipLaunchKernelGGL(combine_send_kernel, dim3(args.max_rows),
                       dim3(block_for_chunks(args.row_bytes / 16)), 0, stream, args, ws, st);
    return hipGetLastError();
}

hipError_t launch_combine_recv(const CombineRecvArgs &args, const Workspace &ws, const Staging &st,
                               uint32_t in_dtype, uint32_t out_dtype, hipStream_t stream) {
    CombArgs ca;
    std::memset(&ca, 0, sizeof ca);
    ca.dst[args.rank] = args.dst;
    for (uint32_t r = 0; r <= (uint32_t)kMaxWorld; ++r) {
        ca.token_start[r] = r <= args.rank ? 0 : args.dst.num_tokens;
    }
    ca.hidden_dim = args.hidden_dim;
    ca.accumulate = args.accumulate;
    ca.staged_base = st.comb_buf;
    ca.staged_stride = st.comb_stride;
    return launch_combine_gather(ca, ws, in_dtype, out_dtype, args.dst.num_tokens, stream);
}

}  // namespace a2a
