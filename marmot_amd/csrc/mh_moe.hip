// MoE on the HIP backend: router helpers (top-k, softmax over the selected logits) and the grouped
// expert FFN: route sort -> shared activation quantization -> grouped gate/up matvec -> SwiGLU + requantize ->
// grouped down matvec -> weighted combine in the reference's accumulation order.
// Compile with -ffp-contract=off.
#include "mh_common.h"

#include <float.h>
#include <stdlib.h>

namespace mh {

constexpr int MOE_ITEM_COLS = 8;   // routes per grouped-matvec work item
constexpr int MOE_MAX_EXPERTS = 1024;
constexpr int MOE_MAX_TOPK = 64;

// ------------------------------------------------------------------ top-k (cpu_topk_impl, moe_ops.c:789-889)
// One thread per row; insertion into a k-long sorted list, ties to the lower index — the same comparisons as the
// reference, so values and indices are identical.
__global__ __launch_bounds__(64) void k_topk(const float *__restrict__ x, size_t rows, size_t cols, size_t k,
                                             float *__restrict__ values, int32_t *__restrict__ indices) {
    const size_t row = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= rows) {
        return;
    }
    float *bv = values + row * k;
    int32_t *bi = indices + row * k;
    for (size_t i = 0; i < k; ++i) {
        bv[i] = -FLT_MAX;
        bi[i] = -1;
    }
    for (size_t col = 0; col < cols; ++col) {
        const float v = x[row * cols + col];
        size_t pos = k;
        for (size_t i = 0; i < k; ++i) {
            const bool better = v > bv[i];
            const bool same = v == bv[i] && (int32_t)col < bi[i];
            if (better || same) {
                pos = i;
                break;
            }
        }
        if (pos == k) {
            continue;
        }
        for (size_t i = k - 1; i > pos; --i) {
            bv[i] = bv[i - 1];
            bi[i] = bi[i - 1];
        }
        bv[pos] = v;
        bi[pos] = (int32_t)col;
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
};

__global__ __launch_bounds__(256) void k_moe_route(const RouteArgs a) {
    __shared__ int counts[MOE_MAX_EXPERTS];
    __shared__ int cursor[MOE_MAX_EXPERTS];
    const int routes = a.T * a.k;
    const int tid = threadIdx.x;
    for (int e = tid; e < a.E; e += blockDim.x) {
        counts[e] = 0;
    }
    __syncthreads();
    for (int r = tid; r < routes; r += blockDim.x) {
        const int id = a.topk_ids[r];
        if (id < 0 || id >= a.E) {
            *a.error_flag = 1;
        } else {
            atomicAdd(&counts[id], 1);
        }
    }
    __syncthreads();
    if (tid == 0) {
        int prefix = 0;
        int n = 0;
        auto place = [&](int e) {
            const int c = counts[e];
            cursor[e] = prefix;
            for (int j = 0; j < c; j += MOE_ITEM_COLS) {
                a.items[n++] = make_int4(e, prefix + j, (c - j) < MOE_ITEM_COLS ? (c - j) : MOE_ITEM_COLS, 0);
            }
            prefix += c;
        };
        if (a.decode_order) {
            // first-appearance order over routes in token-then-slot order; counts[] doubles as "seen" marker
            for (int r = 0; r < routes; ++r) {
                const int id = a.topk_ids[r];
                if (id < 0 || id >= a.E || counts[id] <= 0) {
                    continue;
                }
                place(id);
                counts[id] = -counts[id];
            }
            for (int e = 0; e < a.E; ++e) {
                counts[e] = counts[e] < 0 ? -counts[e] : counts[e];
            }
        } else {
            for (int e = 0; e < a.E; ++e) {
                if (counts[e] != 0) {
                    place(e);
                }
            }
        }
        *a.n_items = n;
    }
    __syncthreads();
    // stable fill by the first wavefront, 64 routes per round in route order
    const int lane = tid & 63;
    for (int base = 0; base < routes; base += 64) {
        if (tid < 64) {
            const int r = base + lane;
            int id = -1;
            if (r < routes) {
                id = a.topk_ids[r];
                if (id < 0 || id >= a.E) {
                    id = -1;
                }
            }
            int rank = 0, cnt = 0;
#pragma unroll
            for (int j = 0; j < 64; ++j) {
                const int idj = __builtin_amdgcn_readlane(id, j);
                const bool same = idj == id;
                cnt += same ? 1 : 0;
                rank += (same && j < lane) ? 1 : 0;
            }
            if (id >= 0) {
                const int pos = cursor[id] + rank;
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
                a.route_pos[r] = pos;
            } else if (r < routes) {
                a.route_pos[r] = -1;
            }
            __builtin_amdgcn_s_waitcnt(0);  // this round's cursor reads are complete before the update below
            if (id >= 0 && rank == cnt - 1) {
                cursor[id] += cnt;
            }
        }
        __syncthreads();
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
    const size_t t = blockIdx.x;
    if (threadIdx.x == 0) {
        int n = 0;
        for (int s = 0; s < k; ++s) {
            const int p = route_pos[t * k + s];
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
        for (int j = 0; j < n; ++j) {
            wts[j] = sorted_weights[pos[j]];
        }
        npos = n;
    }
    __syncthreads();
    const int n = npos;
    for (size_t h = threadIdx.x; h < H; h += blockDim.x) {
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
    hipLaunchKernelGGL(k_topk, dim3((unsigned)((rows + 63) / 64)), dim3(64), 0, dev->stream, d_x, rows, cols, k,
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

int marmot_hip_moe_experts(marmot_hip_device_t *dev, const float *d_hidden, size_t T, size_t H, size_t F, size_t E,
                           size_t k_per_token, int kind_gate_up, int kind_down, const void *d_gate, const void *d_up,
                           const void *d_down, const int32_t *d_topk_ids, const float *d_topk_weights,
                           float weights_scale, int router_weight_policy, int ffn_type, float *d_out) {
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
    const size_t max_items = routes < E + routes / MOE_ITEM_COLS ? routes : E + routes / MOE_ITEM_COLS;
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
    int *flags = (int *)(base + o_flags);  // [0] = number of items, [1] = error flag
    float *gate_out = (float *)(base + o_gate);
    float *up_out = (float *)(base + o_up);
    float *route_down = (float *)(base + o_down);

    extern int marmot_hip_fill_bytes_internal(marmot_hip_device_t *, void *, int, size_t);
    st = marmot_hip_fill_bytes_internal(dev, flags, 0, 2 * sizeof(int));
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }

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
    hipLaunchKernelGGL(k_moe_route, dim3(1), dim3(256), 0, dev->stream, ra);
    MH_HIP(hipGetLastError());

    // hidden states are quantized once per token; routes refer to them through sorted_tokens
    st = launch_quantize_act_soa(dev, act_gu, d_hidden, MARMOT_HIP_DTYPE_F32, T, H, hidden_q);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    const size_t gu_stride = F * ((H + bv_gu - 1) / bv_gu) * block_bytes(kind_gate_up);
    const size_t dn_stride = H * ((F + bv_dn - 1) / bv_dn) * block_bytes(kind_down);
    st = launch_matvec_grouped(dev, kind_gate_up, d_gate, d_up, gu_stride, hidden_q, sorted_tokens, items, flags,
                               max_items, H, F, gate_out, up_out);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    st = launch_quantize_glu_soa(dev, act_dn, gate_out, up_out, ffn_type == MARMOT_HIP_FFN_GEGLU, routes, F, fused_q);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    st = launch_matvec_grouped(dev, kind_down, d_down, nullptr, dn_stride, fused_q, nullptr, items, flags, max_items, F,
                               H, route_down, nullptr);
    if (st != MARMOT_HIP_SUCCESS) {
        return st;
    }
    hipLaunchKernelGGL(k_moe_combine, dim3((unsigned)T), dim3(256), 0, dev->stream, route_down, sorted_weights,
                       route_pos, (int)k_per_token, H, d_out);
    MH_HIP(hipGetLastError());
    set_route("moe_experts_grouped");

    // Expert ids are validated on the device; reading the flag needs a stream synchronization, which is skipped
    // while the stream is being captured into a graph or when MARMOT_HIP_MOE_NO_VALIDATE is set.
    if (!dev->capturing && getenv("MARMOT_HIP_MOE_NO_VALIDATE") == nullptr) {
        int host_flag = 0;
        MH_HIP(hipMemcpyAsync(&host_flag, flags + 1, sizeof(int), hipMemcpyDeviceToHost, dev->stream));
        MH_HIP(hipStreamSynchronize(dev->stream));
        if (host_flag != 0) {
            return set_error(MARMOT_HIP_ERROR_INVALID_ARGUMENT, "MoE expert id is out of range");
        }
    }
    return MARMOT_HIP_SUCCESS;
}

} // extern "C"
