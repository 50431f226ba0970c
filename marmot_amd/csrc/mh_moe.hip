// MoE on the HIP backend: router helpers (top-k, softmax over the selected logits) and the grouped
// expert FFN: route sort -> shared activation quantization -> grouped gate/up matvec -> SwiGLU + requantize ->
// grouped down matvec -> weighted combine in the reference's accumulation order.
// Compile with -ffp-contract=off.
#include "mh_common.h"

#include <float.h>
#include <stdlib.h>

namespace mh {

constexpr int MOE_ITEM_COLS = 8;   // routes per grouped work item (16 or 32 when experts see many routes, see moe_item_cols)
constexpr int MOE_MAX_EXPERTS = 1024;
constexpr int MOE_MAX_TOPK = 64;

// ------------------------------------------------------------------ top-k (cpu_topk_impl, moe_ops.c:789-889)
// The reference inserts the columns in ascending order into a k-long list sorted by value, a new value going in
// front of the first strictly smaller one: the result is the first k columns under the total order (value
// descending, column ascending) among the values greater than -FLT_MAX; NaNs never compare true and are skipped;
// unfilled slots keep (-FLT_MAX, -1). One wavefront per row selects that sequence directly: round r finds the
// largest element that comes strictly after the previous pick in the same order.
__global__ __launch_bounds__(256) void k_topk(const float *__restrict__ x, size_t rows, size_t cols, size_t k,
                                              float *__restrict__ values, int32_t *__restrict__ indices) {
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= rows) {
        return;  // uniform per wavefront
    }
    const float *in = x + row * cols;
    float last_v = INFINITY;
    int last_i = -1;
    bool done = false;
    for (size_t r = 0; r < k; ++r) {
        float bv = -FLT_MAX;
        int bi = -1;
        if (!done) {
            for (size_t col = lane; col < cols; col += 64) {
                const float v = in[col];
                const bool after_last = v < last_v || (v == last_v && (int)col > last_i);
                if (after_last && v > bv) {  // ascending columns: an equal later value never replaces
                    bv = v;
                    bi = (int)col;
                }
            }
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) {
                const float ov = __shfl_xor(bv, d, 64);
                const int oi = __shfl_xor(bi, d, 64);
                if (ov > bv || (ov == bv && oi >= 0 && oi < bi)) {
                    bv = ov;
                    bi = oi;
                }
            }
            if (bi < 0) {
                done = true;
            } else {
                last_v = bv;
                last_i = bi;
            }
        }
        if (lane == 0) {
            values[row * k + r] = bv;
            indices[row * k + r] = bi;
        }
    }
}

// softmax over each row of k selected logits: max-subtract, expf, in-order sum, divide
__global__ __launch_bounds__(64) void k_softmax_rows(const float *__restrict__ x, size_t rows, size_t k,
                                                     float *__restrict__ out) {
    const size_t row = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= rows) {
        return;
    }
    const float *in = x + row * k;
    float *o = out + row * k;
    float mx = in[0];
    for (size_t i = 1; i < k; ++i) {
        mx = in[i] > mx ? in[i] : mx;
    }
    float sum = 0.0f;
    for (size_t i = 0; i < k; ++i) {
        const float e = expf(in[i] - mx);
        o[i] = e;
        sum += e;
    }
    for (size_t i = 0; i < k; ++i) {
        o[i] = o[i] / sum;
    }
}

// ------------------------------------------------------------------ route sort
// cpu_moe_execute_grouped (moe_ops.c:905-974): count routes per expert, exclusive prefix over experts, then a
// stable fill in token-then-slot order. `decode_order` reproduces cpu_moe_execute_decode (moe_ops.c:643-717), where
// experts are laid out in order of first appearance instead of ascending id. Also cuts every expert's segment into
// work items of up to MOE_ITEM_COLS routes for the grouped matvec.
struct RouteArgs {
    const int32_t *topk_ids;      // [T, k]
    const float *topk_weights;    // [T, k]
    uint32_t *sorted_tokens;      // [routes]
    float *sorted_weights;        // [routes]
    int *route_pos;               // [T, k] position of each (token, slot) in the sorted order
    int4 *items;                  // work items
    int *n_items;
    int *error_flag;              // set to 1 when an expert id is out of range
    int T, k, E;
    float weights_scale;
    int renormalize;
    int decode_order;
    int item_cols;                // routes per work item: 8, 16 or 32
};

constexpr int MOE_ROUTE_LDS = 4096;    // routes whose ids and positions are kept in LDS
constexpr int MOE_ROUTE_WAVES = 8;     // wavefronts of the route kernel; each fills one contiguous chunk of routes

// exclusive prefix sum over the 64 lanes of a wavefront; *total receives the sum over all lanes
__device__ __forceinline__ int wave_excl_scan(int v, int lane, int *total) {
    int incl = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d, 64);
        if (lane >= d) {
            incl += up;
        }
    }
    *total = __shfl(incl, 63, 64);
    return incl - v;
}

// rank = number of lower lanes holding the same id, cnt = number of lanes holding it
__device__ __forceinline__ void wave_rank(int id, int lane, int *rank, int *cnt) {
    int rk = 0, c = 0;
#pragma unroll
    for (int j = 0; j < 64; ++j) {
        const int idj = __builtin_amdgcn_readlane(id, j);
        const bool same = idj == id;
        c += same ? 1 : 0;
        rk += (same && j < lane) ? 1 : 0;
    }
    *rank = rk;
    *cnt = c;
}

__device__ __forceinline__ void route_emit(const RouteArgs &a, int r, int pos) {
    a.route_pos[r] = pos;
    if (pos < 0) {
        return;
    }
    const int t = r / a.k;
    float norm = a.weights_scale;
    if (a.renormalize) {
        float wsum = 0.0f;
        for (int s = 0; s < a.k; ++s) {
            wsum += a.topk_weights[t * a.k + s];
        }
        norm = wsum > FLT_MIN ? a.weights_scale / wsum : 0.0f;
    }
    a.sorted_tokens[pos] = (uint32_t)t;
    a.sorted_weights[pos] = a.topk_weights[r] * norm;
}

__global__ __launch_bounds__(MOE_ROUTE_WAVES * 64) void k_moe_route(const RouteArgs a) {
    warm_kernel_arguments<sizeof(RouteArgs), sizeof(RouteArgs)>();
    __shared__ int counts[MOE_MAX_EXPERTS];
    __shared__ int wcount[MOE_ROUTE_WAVES][MOE_MAX_EXPERTS];  // per chunk: routes of each expert, then its cursor
    __shared__ int ids_l[MOE_ROUTE_LDS];  // expert id of each route (-1 = invalid), later its sorted position
    const int routes = a.T * a.k;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    if (a.decode_order) {
        // At most 64 routes: one wavefront, one round. Experts are laid out in order of first appearance, so the
        // segment of an expert starts at the number of routes whose expert appeared earlier: an exclusive scan of
        // the expert's route count over the lanes that hold a first appearance.
        if (wave != 0) {
            return;
        }
        int id = -1;
        if (lane < routes) {
            id = a.topk_ids[lane];
            if (id < 0 || id >= a.E) {
                id = -1;
            }
        }
        const unsigned long long bad = __ballot(lane < routes && id < 0);
        int rank, cnt;
        wave_rank(id, lane, &rank, &cnt);
        const bool first = id >= 0 && rank == 0;
        int total, n_items;
        const int seg = wave_excl_scan(first ? cnt : 0, lane, &total);
        const int item0 = wave_excl_scan(first ? (cnt + a.item_cols - 1) / a.item_cols : 0, lane, &n_items);
        if (first) {
            counts[id] = seg;
            int n = item0;
            for (int j = 0; j < cnt; j += a.item_cols) {
                a.items[n++] = make_int4(id, seg + j, (cnt - j) < a.item_cols ? (cnt - j) : a.item_cols, 0);
            }
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the segment starts are in LDS (same wavefront)
        if (lane < routes) {
            route_emit(a, lane, id >= 0 ? counts[id] + rank : -1);
        }
        if (lane == 0) {
            *a.n_items = n_items;
            *a.error_flag = bad != 0 ? 1 : 0;
        }
        return;
    }

    const bool in_lds = routes <= MOE_ROUTE_LDS;
    for (int e = tid; e < a.E; e += blockDim.x) {
#pragma unroll
        for (int w = 0; w < MOE_ROUTE_WAVES; ++w) {
            wcount[w][e] = 0;
        }
    }
    if (tid == 0) {
        *a.error_flag = 0;
    }
    __syncthreads();
    // chunk of wavefront w: routes [w * chunk, (w + 1) * chunk), a multiple of 64
    const int chunk = ((routes + MOE_ROUTE_WAVES * 64 - 1) / (MOE_ROUTE_WAVES * 64)) * 64;
    const int r_begin = wave * chunk;
    const int r_end = r_begin + chunk < routes ? r_begin + chunk : routes;
    for (int r = r_begin + lane; r < r_end; r += 64) {
        int id = a.topk_ids[r];
        if (id < 0 || id >= a.E) {
            *a.error_flag = 1;
            id = -1;
        } else {
            atomicAdd(&wcount[wave][id], 1);
        }
        if (in_lds) {
            ids_l[r] = id;
        }
    }
    __syncthreads();
    for (int e = tid; e < a.E; e += blockDim.x) {
        int c = 0;
#pragma unroll
        for (int w = 0; w < MOE_ROUTE_WAVES; ++w) {
            c += wcount[w][e];
        }
        counts[e] = c;
    }
    __syncthreads();
    // exclusive prefix over experts in ascending id and the work items of every expert: lane l of the first
    // wavefront owns the experts [l * per, (l + 1) * per)
    if (wave == 0) {
        const int per = (a.E + 63) / 64;
        const int e0 = lane * per;
        const int e1 = e0 + per < a.E ? e0 + per : a.E;
        int c_sum = 0, i_sum = 0;
        for (int e = e0; e < e1; ++e) {
            const int c = counts[e];
            c_sum += c;
            i_sum += (c + a.item_cols - 1) / a.item_cols;
        }
        int total, n_items;
        int prefix = wave_excl_scan(c_sum, lane, &total);
        int n = wave_excl_scan(i_sum, lane, &n_items);
        for (int e = e0; e < e1; ++e) {
            const int c = counts[e];
            counts[e] = prefix;  // from here on: start of the expert's segment
            for (int j = 0; j < c; j += a.item_cols) {
                a.items[n++] = make_int4(e, prefix + j, (c - j) < a.item_cols ? (c - j) : a.item_cols, 0);
            }
            prefix += c;
        }
        if (lane == 0) {
            *a.n_items = n_items;
        }
    }
    __syncthreads();
    // cursor of chunk w for expert e: segment start + routes of e in earlier chunks
    for (int e = tid; e < a.E; e += blockDim.x) {
        int run = counts[e];
#pragma unroll
        for (int w = 0; w < MOE_ROUTE_WAVES; ++w) {
            const int c = wcount[w][e];
            wcount[w][e] = run;
            run += c;
        }
    }
    __syncthreads();
    // Stable fill, every wavefront over its own chunk, 64 routes per round in route order: a route's position is its
    // expert's cursor plus the number of earlier lanes of the round with the same expert.
    int *cursor = wcount[wave];
    for (int base = r_begin; base < r_end; base += 64) {
        const int r = base + lane;
        int id = -1;
        if (r < r_end) {
            if (in_lds) {
                id = ids_l[r];
            } else {
                id = a.topk_ids[r];
                if (id < 0 || id >= a.E) {
                    id = -1;
                }
            }
        }
        int rank, cnt;
        wave_rank(id, lane, &rank, &cnt);
        int pos = -1;
        if (id >= 0) {
            pos = cursor[id] + rank;
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // this round's cursor reads are complete before the update below
        if (id >= 0 && rank == cnt - 1) {
            cursor[id] += cnt;
        }
        if (r < r_end) {
            route_emit(a, r, pos);
        }
    }
}

// ------------------------------------------------------------------ weighted combine
// out[t, :] = sum over the token's routes, in ascending sorted position (moe_ops.c:1034-1042), of
// weight * down_row; tokens without a valid route get zeros (moe_ops.c:944-947, 984-986).
__global__ __launch_bounds__(256) void k_moe_combine(const float *__restrict__ route_down,
                                                     const float *__restrict__ sorted_weights,
                                                     const int *__restrict__ route_pos, int k, size_t H,
                                                     float *__restrict__ out) {
    __shared__ int pos[MOE_MAX_TOPK];
    __shared__ float wts[MOE_MAX_TOPK];
    __shared__ int npos;
    __shared__ int raw[MOE_MAX_TOPK];
    const size_t t = blockIdx.x;
    if ((int)threadIdx.x < k) {
        raw[threadIdx.x] = route_pos[t * k + threadIdx.x];
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int n = 0;
        for (int s = 0; s < k; ++s) {
            const int p = raw[s];
            if (p < 0) {
                continue;
            }
            int j = n++;
            while (j > 0 && pos[j - 1] > p) {
                pos[j] = pos[j - 1];
                --j;
            }
            pos[j] = p;
        }
        npos = n;
    }
    __syncthreads();
    if ((int)threadIdx.x < npos) {
        wts[threadIdx.x] = sorted_weights[pos[threadIdx.x]];
    }
    __syncthreads();
    const int n = npos;
    // blockIdx.y selects a slab of 256 columns
    const size_t h = (size_t)blockIdx.y * blockDim.x + threadIdx.x;
    if (h < H) {
        float acc = 0.0f;
        for (int j = 0; j < n; ++j) {
            acc += wts[j] * route_down[(size_t)pos[j] * H + h];
        }
        out[t * H + h] = acc;
    }
}

static inline size_t round256(size_t v) {
    return (v + 255) & ~(size_t)255;
}

} // namespace mh

using namespace mh;

extern "C" {

int marmot_hip_topk(marmot_hip_device_t *dev, const float *d_x, size_t rows, size_t cols, size_t k, float *d_values,
                    int32_t *d_indices) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_x == nullptr || d_values == nullptr || d_indices == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "TopK descriptor is incomplete");
    }
    if (k == 0 || k > cols) {
        return set_error(MARMOT_HIP_ERROR_DIMENSION_MISMATCH, "TopK shapes do not match");
    }
    if (rows == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    hipLaunchKernelGGL(k_topk, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, dev->stream, d_x, rows, cols, k,
                       d_values, d_indices);
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

int marmot_hip_softmax_rows(marmot_hip_device_t *dev, const float *d_x, size_t rows, size_t k, float *d_out) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_x == nullptr || d_out == nullptr || k == 0) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "softmax_rows: bad argument");
    }
    if (rows == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    hipLaunchKernelGGL(k_softmax_rows, dim3((unsigned)((rows + 63) / 64)), dim3(64), 0, dev->stream, d_x, rows, k,
                       d_out);
    MH_HIP(hipGetLastError());
    return MARMOT_HIP_SUCCESS;
}

} // extern "C"

// One body for marmot_hip_moe_experts and its stage-probing variant. `probe` (may be null) names device buffers that
// receive the intermediate arrays, and optionally the packed activations the down projection reads instead of the
// ones this call quantized.
static int moe_experts_impl(marmot_hip_device_t *dev, const float *d_hidden, size_t T, size_t H, size_t F, size_t E,
                            size_t k_per_token, int kind_gate_up, int kind_down, const void *d_gate, const void *d_up,
                            const void *d_down, const int32_t *d_topk_ids, const float *d_topk_weights,
                            float weights_scale, int router_weight_policy, int ffn_type, float *d_out,
                            const marmot_hip_moe_probe_t *probe) {
    if (dev == nullptr) {
        return set_error(MARMOT_HIP_ERROR_DEVICE_NOT_AVAILABLE, "HIP device is not initialised");
    }
    if (d_hidden == nullptr || d_gate == nullptr || d_up == nullptr || d_down == nullptr || d_topk_ids == nullptr ||
        d_topk_weights == nullptr || d_out == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "MoE experts requires non-null context and tensors");
    }
    if (router_weight_policy < 0 || router_weight_policy > MARMOT_HIP_ROUTER_RENORMALIZE_SELECTED) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "MoE experts requires a valid router weight policy");
    }
    if (ffn_type != MARMOT_HIP_FFN_SWIGLU && ffn_type != MARMOT_HIP_FFN_GEGLU) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "MoE experts currently supports SwiGLU and GeGLU only");
    }
    const size_t bv_gu = block_values(kind_gate_up), bv_dn = block_values(kind_down);
    if (bv_gu == 0 || bv_dn == 0 || kind_gate_up == MARMOT_HIP_KIND_Q8_K || kind_down == MARMOT_HIP_KIND_Q8_K) {
        return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "MoE experts: unsupported expert quant kinds %d / %d",
                         kind_gate_up, kind_down);
    }
    if (E == 0 || E > (size_t)MOE_MAX_EXPERTS || k_per_token == 0 || k_per_token > (size_t)MOE_MAX_TOPK || H == 0 ||
        F == 0) {
        return set_error(MARMOT_HIP_ERROR_DIMENSION_MISMATCH, "MoE expert tensor shapes do not match");
    }
    if (T == 0) {
        return MARMOT_HIP_SUCCESS;
    }
    MH_HIP(hipSetDevice(dev->device_index));

    const size_t routes = T * k_per_token;
    // Routes per work item. A work item streams its expert's rows once for its routes, so prompts, where an expert
    // sees dozens of routes, take wider items (the small-batch kernels on the int8 matrix cores hold 16 or 32 activation
    // rows per pass; the dot-product kernel of the 32-value formats holds 8): E = 128, top 8, 512 tokens: 325 us with 8.
    const bool mmq_gu = mmq_grouped_supported(dev, kind_gate_up, H), mmq_dn = mmq_grouped_supported(dev, kind_down, F);
    const auto q45 = [](int kind) { return kind == MARMOT_HIP_KIND_Q4_K || kind == MARMOT_HIP_KIND_Q5_K; };
    size_t item_cols = MOE_ITEM_COLS;
    if (mmq_gu && mmq_dn && routes >= 12 * E) {
        item_cols = (routes >= 24 * E && q45(kind_gate_up) && q45(kind_down)) ? 32 : 16;
    }
    const size_t max_items = routes < E + routes / item_cols ? routes : E + routes / item_cols;
    const int act_gu = is_k_quant(kind_gate_up) ? MARMOT_HIP_KIND_Q8_K : MARMOT_HIP_KIND_Q8_0;
    const int act_dn = is_k_quant(kind_down) ? MARMOT_HIP_KIND_Q8_K : MARMOT_HIP_KIND_Q8_0;

    // workspace carve-up
    size_t off = 0;
    auto take = [&](size_t bytes) {
        const size_t o = off;
        off += round256(bytes);
        return o;
    };
    const size_t o_hidden_q = take(act_scratch_layout(act_gu, T, H, nullptr, nullptr));
    const size_t o_fused_q = take(act_scratch_layout(act_dn, routes, F, nullptr, nullptr));
    const size_t o_tokens = take(routes * sizeof(uint32_t));
    const size_t o_weights = take(routes * sizeof(float));
    const size_t o_pos = take(routes * sizeof(int));
    const size_t o_items = take((max_items + 1) * sizeof(int4));
    const size_t o_flags = take(2 * sizeof(int));
    const size_t o_gate = take(routes * F * sizeof(float));
    const size_t o_up = take(routes * F * sizeof(float));
    const size_t o_down = take(routes * H * sizeof(float));
    void *ws = nullptr;
    int st = workspace_reserve(dev, off, &ws);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    uint8_t *base = (uint8_t *)ws;
    ActScratch hidden_q, fused_q;
    act_scratch_layout(act_gu, T, H, base + o_hidden_q, &hidden_q);
    act_scratch_layout(act_dn, routes, F, base + o_fused_q, &fused_q);
    uint32_t *sorted_tokens = (uint32_t *)(base + o_tokens);
    float *sorted_weights = (float *)(base + o_weights);
    int *route_pos = (int *)(base + o_pos);
    int4 *items = (int4 *)(base + o_items);
    int *flags = (int *)(base + o_flags);  // [0] = number of items, [1] = error flag; both set by the route kernel
    float *gate_out = (float *)(base + o_gate);
    float *up_out = (float *)(base + o_up);
    float *route_down = (float *)(base + o_down);

    RouteArgs ra;
    ra.topk_ids = d_topk_ids;
    ra.topk_weights = d_topk_weights;
    ra.sorted_tokens = sorted_tokens;
    ra.sorted_weights = sorted_weights;
    ra.route_pos = route_pos;
    ra.items = items;
    ra.n_items = flags;
    ra.error_flag = flags + 1;
    ra.T = (int)T;
    ra.k = (int)k_per_token;
    ra.E = (int)E;
    ra.weights_scale = weights_scale;
    ra.renormalize = router_weight_policy == MARMOT_HIP_ROUTER_RENORMALIZE_SELECTED;
    // cpu_moe_should_use_decode_path (moe_ops.c:417-424)
    ra.decode_order = (T <= 4 && routes <= 64) ? 1 : 0;
    ra.item_cols = (int)item_cols;
    hipLaunchKernelGGL(k_moe_route, dim3(1), dim3(MOE_ROUTE_WAVES * 64), 0, dev->stream, ra);
    MH_HIP(hipGetLastError());

    // hidden states are quantized once per token; routes refer to them through sorted_tokens
    st = launch_quantize_act_soa(dev, act_gu, d_hidden, MARMOT_HIP_DTYPE_F32, T, H, hidden_q);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    const size_t gu_stride = F * ((H + bv_gu - 1) / bv_gu) * block_bytes(kind_gate_up);
    const size_t dn_stride = H * ((F + bv_dn - 1) / bv_dn) * block_bytes(kind_down);
    // Q4_K / Q6_K experts run on the int8 matrix cores, the 32-value formats on the dot-product matvec
    st = mmq_gu ? launch_mmq_grouped(dev, kind_gate_up, d_gate, d_up, gu_stride, hidden_q, sorted_tokens, items, flags,
                                     max_items, H, F, gate_out, up_out, (int)item_cols)
                : launch_matvec_grouped(dev, kind_gate_up, d_gate, d_up, gu_stride, hidden_q, sorted_tokens, items, flags,
                                        max_items, H, F, gate_out, up_out);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    st = launch_quantize_glu_soa(dev, act_dn, gate_out, up_out, ffn_type == MARMOT_HIP_FFN_GEGLU, routes, F, fused_q);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    if (probe != nullptr) {
        const size_t fused_bytes = act_scratch_layout(act_dn, routes, F, nullptr, nullptr);
        const struct {
            void *dst;
            const void *src;
            size_t bytes;
        } copies[] = {
            {probe->d_sorted_tokens, sorted_tokens, routes * sizeof(uint32_t)},
            {probe->d_route_pos, route_pos, routes * sizeof(int)},
            {probe->d_gate_out, gate_out, routes * F * sizeof(float)},
            {probe->d_up_out, up_out, routes * F * sizeof(float)},
            {probe->d_fused_packed, base + o_fused_q, fused_bytes},
        };
        for (const auto &c : copies) {
            if (c.dst != nullptr) {
                MH_HIP(hipMemcpyAsync(c.dst, c.src, c.bytes, hipMemcpyDeviceToDevice, dev->stream));
            }
        }
        if (probe->d_fused_override != nullptr) {
            MH_HIP(hipMemcpyAsync(base + o_fused_q, probe->d_fused_override, fused_bytes, hipMemcpyDeviceToDevice,
                                  dev->stream));
        }
    }
    st = mmq_dn ? launch_mmq_grouped(dev, kind_down, d_down, nullptr, dn_stride, fused_q, nullptr, items, flags, max_items,
                                     F, H, route_down, nullptr, (int)item_cols)
                : launch_matvec_grouped(dev, kind_down, d_down, nullptr, dn_stride, fused_q, nullptr, items, flags,
                                        max_items, F, H, route_down, nullptr);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    hipLaunchKernelGGL(k_moe_combine, dim3((unsigned)T, (unsigned)((H + 255) / 256)), dim3(256), 0, dev->stream,
                       route_down, sorted_weights, route_pos, (int)k_per_token, H, d_out);
    MH_HIP(hipGetLastError());
    set_route("moe_experts_grouped");

    // Expert ids are validated on the device; reading the flag needs a stream synchronization, which is skipped
    // while the stream is being captured into a graph or when the device object was created with
    // MARMOT_HIP_MOE_NO_VALIDATE set.
    if (!dev->capturing && !dev->knobs.moe_no_validate) {
        int host_flag = 0;
        MH_HIP(hipMemcpyAsync(&host_flag, flags + 1, sizeof(int), hipMemcpyDeviceToHost, dev->stream));
        MH_HIP(hipStreamSynchronize(dev->stream));
        if (host_flag != 0) {
            return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "MoE expert id is out of range");
        }
    }
    return MARMOT_HIP_SUCCESS;
}

extern "C" {

int marmot_hip_moe_experts(marmot_hip_device_t *dev, const float *d_hidden, size_t T, size_t H, size_t F, size_t E,
                           size_t k_per_token, int kind_gate_up, int kind_down, const void *d_gate, const void *d_up,
                           const void *d_down, const int32_t *d_topk_ids, const float *d_topk_weights,
                           float weights_scale, int router_weight_policy, int ffn_type, float *d_out) {
    return moe_experts_impl(dev, d_hidden, T, H, F, E, k_per_token, kind_gate_up, kind_down, d_gate, d_up, d_down,
                            d_topk_ids, d_topk_weights, weights_scale, router_weight_policy, ffn_type, d_out, nullptr);
}

int marmot_hip_moe_experts_probe(marmot_hip_device_t *dev, const float *d_hidden, size_t T, size_t H, size_t F,
                                 size_t E, size_t k_per_token, int kind_gate_up, int kind_down, const void *d_gate,
                                 const void *d_up, const void *d_down, const int32_t *d_topk_ids,
                                 const float *d_topk_weights, float weights_scale, int router_weight_policy,
                                 int ffn_type, float *d_out, const marmot_hip_moe_probe_t *probe) {
    if (probe == nullptr) {
        return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "MoE experts probe requires a probe description");
    }
    if (dev != nullptr && dev->capturing) {
        return set_error(MARMOT_HIP_ERROR_INVALID_OPERATION, "MoE experts probe cannot be captured into a graph");
    }
    return moe_experts_impl(dev, d_hidden, T, H, F, E, k_per_token, kind_gate_up, kind_down, d_gate, d_up, d_down,
                            d_topk_ids, d_topk_weights, weights_scale, router_weight_policy, ffn_type, d_out, probe);
}

} // extern "C"
