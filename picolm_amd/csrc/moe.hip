// A routed feed-forward (mixers.h): every row picks a few experts by its router logits and only
// their weights are read.  Three kernels: the pick; the picked experts' hidden units (a workgroup
// per (row, pick, 16 hidden units)); the down products with the weighted sum over a row's picks (a
// workgroup per (row, 16 outputs)), so that a row's result is added up in one place and in a fixed
// order.  A wave takes one weight row at a time, 16 bytes a lane, against the row's input in LDS.
// Logits, picks, weights, hidden units and sums are float.
//
// A prompt (64 rows and more, bfloat16) goes through the matrix cores instead: the (row, pick) pairs
// are sorted by expert in one workgroup, a workgroup takes 128 pairs of one expert by 64 hidden units
// (or outputs) through LDS with v_mfma_f32_32x32x16_bf16; the hidden units are rounded to bfloat16
// once, as every product's input is; a last kernel adds a row's picks up in their order.  Which
// pairs share a tile changes no pair's result.
#include "mixers.h"

#include "api.h"
#include "common.h"
#include "gemm_mfma.h"

#define VIEW_REQUIRE(who, v)                                                                                      \
    PICOLM_REQUIRE((v) && (v)->struct_bytes == (int32_t)sizeof(picolm_step_view), "%s: the step view is of another version", who)

static inline int elem_bytes(int dt) { return dt == PICOLM_F32 ? 4 : 2; }

// ---- the pick --------------------------------------------------------------------------------------
// a thread a row; the picks come out in the order (logit falling, index rising)
__global__ void route_top_kernel(const float* __restrict__ logits, int in_stride, const float* __restrict__ bias, int32_t* __restrict__ out, int E,
                                 int top, int n_rows, int scoring, float scale) {
    const int row = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= n_rows) return;
    const float* z = logits + (size_t)row * in_stride;
    int32_t* ids = out + (size_t)row * 2 * top;
    float* w = (float*)(ids + top);
    if (scoring == 2) {
        // s = sigmoid of every output; the picks are the largest s + bias, their weights the picked s themselves
        float last_c = INFINITY;
        int last_e = -1;
        for (int k = 0; k < top; ++k) {
            float best = -INFINITY, best_s = 0.f;
            int be = -1;
            for (int e = 0; e < E; ++e) {
                const float se = 1.f / (1.f + expf(-z[e])), ce = se + (bias ? bias[e] : 0.f);
                const bool after_last = ce < last_c || (ce == last_c && e > last_e);
                if (after_last && (be < 0 || ce > best)) best = ce, be = e, best_s = se;
            }
            if (be < 0) be = k % E, best = -INFINITY, best_s = 0.f;     // (only logits that are no numbers lead here)
            ids[k] = be;
            w[k] = best_s * scale;
            last_c = best, last_e = be;
        }
        return;
    }
    if (scoring == 1) {
        // s = softmax over every output; the picks are the largest s + bias, their weights the picked s over their sum
        float zmax = -INFINITY, den = 0.f;
        for (int e = 0; e < E; ++e) zmax = fmaxf(zmax, z[e]);
        for (int e = 0; e < E; ++e) den += expf(z[e] - zmax);
        float last_c = INFINITY, sum = 0.f;
        int last_e = -1;
        for (int k = 0; k < top; ++k) {
            float best = -INFINITY, best_s = 0.f;
            int be = -1;
            for (int e = 0; e < E; ++e) {
                const float se = expf(z[e] - zmax) / den, ce = se + (bias ? bias[e] : 0.f);
                const bool after_last = ce < last_c || (ce == last_c && e > last_e);
                if (after_last && (be < 0 || ce > best)) best = ce, be = e, best_s = se;
            }
            if (be < 0) be = k % E, best = -INFINITY, best_s = 0.f;     // (only logits that are no numbers lead here)
            ids[k] = be;
            w[k] = best_s;
            sum += best_s;
            last_c = best, last_e = be;
        }
        for (int k = 0; k < top; ++k) w[k] = w[k] / (sum + 1e-20f) * scale;
        return;
    }
    float last_z = INFINITY, first_z = 0.f, sum = 0.f;
    int last_e = -1;
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int be = -1;
        for (int e = 0; e < E; ++e) {
            const float ze = z[e] + (bias ? bias[e] : 0.f);
            const bool after_last = ze < last_z || (ze == last_z && e > last_e);
            if (after_last && (be < 0 || ze > best)) best = ze, be = e;
        }
        if (be < 0) be = k % E, best = -INFINITY;     // (only logits that are no numbers lead here)
        if (k == 0) first_z = best;
        const float p = expf(best - first_z);
        ids[k] = be;
        w[k] = p;
        sum += p;
        last_z = best, last_e = be;
    }
    for (int k = 0; k < top; ++k) w[k] /= sum;
}

extern "C" int picolm_call_route_top(void* user, const picolm_step_view* v) {
    const picolm_route_top_args* a = (const picolm_route_top_args*)user;
    VIEW_REQUIRE("route_top", v);
    PICOLM_REQUIRE(a && v->in && v->out && a->experts > 0 && a->top > 0 && a->top <= a->experts, "route_top: %d picks among %d experts",
                   a ? a->top : 0, a ? a->experts : 0);
    const int in_stride = a->in_stride ? a->in_stride : a->experts;
    PICOLM_REQUIRE(in_stride >= a->experts && v->in_row_bytes >= (int64_t)in_stride * 4 && v->out_row_bytes >= 2 * a->top * 4, "route_top: rows too short");
    PICOLM_REQUIRE(a->scoring >= 0 && a->scoring <= 2, "route_top: scoring %d is not known", a->scoring);
    if (v->rows <= 0) return 0;
    route_top_kernel<<<ceil_div(v->rows, 64), 64, 0, v->stream>>>((const float*)v->in, in_stride, a->bias, (int32_t*)v->out, a->experts, a->top,
                                                                 v->rows, a->scoring, a->scale);
    PICOLM_LAUNCH_CHECK("route_top");
    return 0;
}

// ---- the picked experts ------------------------------------------------------------------------------
// a lane's share of the dot product of a weight row with floats in LDS
template <typename TW> __device__ __forceinline__ float lane_dot(const TW* __restrict__ w, const float* __restrict__ h, int K, int lane);
template <> __device__ __forceinline__ float lane_dot<bf16_t>(const bf16_t* __restrict__ w, const float* __restrict__ h, int K, int lane) {
    float acc = 0.f;
    if (K % 8 == 0) {
        for (int i = lane * 8; i < K; i += WAVE * 8) {
            const uint4 p = *(const uint4*)(w + i);
            const uint32_t u[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc += __uint_as_float(u[j] << 16) * h[i + 2 * j];
                acc += __uint_as_float(u[j] & 0xffff0000u) * h[i + 2 * j + 1];
            }
        }
    } else {
        for (int i = lane; i < K; i += WAVE) acc += bf16_bits_to_f32(w[i]) * h[i];
    }
    return acc;
}
template <> __device__ __forceinline__ float lane_dot<float>(const float* __restrict__ w, const float* __restrict__ h, int K, int lane) {
    float acc = 0.f;
    if (K % 4 == 0) {
        for (int i = lane * 4; i < K; i += WAVE * 4) {
            const float4 p = *(const float4*)(w + i);
            acc += p.x * h[i] + p.y * h[i + 1] + p.z * h[i + 2] + p.w * h[i + 3];
        }
    } else {
        for (int i = lane; i < K; i += WAVE) acc += w[i] * h[i];
    }
    return acc;
}

#define MOE_UNITS 16     // hidden units, or outputs, a workgroup of four waves takes

// what an expert's hidden unit is, from its two products g and u (mixers.h: picolm_routed_experts_args.act)
struct ExpertAct {
    int kind;
    float limit, alpha;
    int weight_on_input;
};
__device__ __forceinline__ float expert_act(const ExpertAct& x, float g, float u) {
    if (x.kind == 1) {
        g = fminf(g, x.limit);
        u = fminf(fmaxf(u, -x.limit), x.limit);
        return g / (1.f + expf(-x.alpha * g)) * (u + 1.f);
    }
    return g / (1.f + expf(-g)) * u;
}

// act[row][pick][f] = silu(W_gate[e][f] . h) * (W_up[e][f] . h); a wave has its four units' eight rows on their way at once
template <typename TW, typename TH>
__global__ __launch_bounds__(256) void expert_hidden_kernel(const TH* __restrict__ h, const int32_t* __restrict__ picks, float* __restrict__ act,
                                                            const TW* __restrict__ gate, const TW* __restrict__ up, int E, int top, int D, int F,
                                                            ExpertAct xa) {
    extern __shared__ float moe_lds[];       // [D]
    const int pair = blockIdx.x, row = pair / top, k = pair % top;
    const int e = picks[(size_t)row * 2 * top + k];
    for (int c = threadIdx.x; c < D; c += blockDim.x) moe_lds[c] = to_f32<TH>(h[(size_t)row * D + c]);
    __syncthreads();
    if (e < 0 || e >= E) return;
    const float on_input = xa.weight_on_input ? ((const float*)(picks + (size_t)row * 2 * top + top))[k] : 1.f;
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int f0 = blockIdx.y * MOE_UNITS + wave * 4;
    float g[4], u[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const size_t w_row = ((size_t)e * F + min(f0 + j, F - 1)) * D;
        g[j] = lane_dot<TW>(gate + w_row, moe_lds, D, lane);
        u[j] = lane_dot<TW>(up + w_row, moe_lds, D, lane);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float gs = wave_sum(g[j]) * on_input, us = wave_sum(u[j]) * on_input;
        if (lane == 0 && f0 + j < F) act[((size_t)row * top + k) * F + f0 + j] = expert_act(xa, gs, us);
    }
}

// out[row][d] (+)= sum_k w[row][k] (W_down[e_k][d] . act[row][k])
// a row's picks that stand for "the input itself": the sum of their weights
__device__ __forceinline__ float identity_weight(const int32_t* ids, const float* w, int top, int E, int identity) {
    float total = 0.f;
    for (int k = 0; k < top; ++k)
        if (ids[k] >= E && ids[k] < E + identity) total += w[k];
    return total;
}

template <typename TW, typename TH>
__global__ __launch_bounds__(256) void expert_down_kernel(const float* __restrict__ act, const int32_t* __restrict__ picks, float* __restrict__ out,
                                                          const TW* __restrict__ down, int E, int top, int D, int F, int adds,
                                                          const TH* __restrict__ h, int identity, int plain_sum) {
    extern __shared__ float moe_lds[];       // [top][F]
    const int row = blockIdx.x;
    for (int c = threadIdx.x; c < top * F; c += blockDim.x) moe_lds[c] = act[(size_t)row * top * F + c];
    __syncthreads();
    const int32_t* ids = picks + (size_t)row * 2 * top;
    const float* w = (const float*)(ids + top);
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int d0 = blockIdx.y * MOE_UNITS + wave * 4;
    float total[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < top; ++k) {
        const int e = ids[k];
        if (e < 0 || e >= E) continue;
        float part[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) part[j] = lane_dot<TW>(down + ((size_t)e * D + min(d0 + j, D - 1)) * F, moe_lds + (size_t)k * F, F, lane);
#pragma unroll
        for (int j = 0; j < 4; ++j) total[j] += (plain_sum ? 1.f : w[k]) * wave_sum(part[j]);
    }
    const float same = identity > 0 ? identity_weight(ids, w, top, E, identity) : 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j)
        if (lane == 0 && d0 + j < D) {
            const size_t at = (size_t)row * D + d0 + j;
            out[at] = (adds ? out[at] : 0.f) + total[j] + (same != 0.f ? same * to_f32<TH>(h[at]) : 0.f);
        }
}

// ---- the same for many rows, on the matrix cores ------------------------------------------------------
#define GM_ROWS 128      // pairs of a tile
#define GM_MAX_EXPERTS 4096

// plan: [0 .. E] where each expert's pairs start in the sorted list, then the sorted pairs (pair = row * top + pick)
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int32_t* __restrict__ picks, int32_t* __restrict__ plan, int E, int top,
                                                        int n_pairs) {
    extern __shared__ int32_t plan_lds[];      // counts, then cursors [E] | starts [E + 1]
    int32_t* counts = plan_lds;
    int32_t* starts = plan_lds + E;
    for (int e = threadIdx.x; e < E; e += blockDim.x) counts[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
        const int e = picks[(size_t)(p / top) * 2 * top + p % top];
        if (e >= 0 && e < E) atomicAdd(&counts[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0;
        for (int e = 0; e < E; ++e) {
            starts[e] = at;
            at += counts[e];
            counts[e] = 0;
        }
        starts[E] = at;
    }
    __syncthreads();
    for (int e = threadIdx.x; e <= E; e += blockDim.x) plan[e] = starts[e];
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
        const int e = picks[(size_t)(p / top) * 2 * top + p % top];
        if (e >= 0 && e < E) plan[E + 1 + starts[e] + atomicAdd(&counts[e], 1)] = p;
    }
}

// the tile of GM_ROWS pairs that a workgroup takes: its expert, and its pairs into LDS (-1 past the expert's last)
__device__ __forceinline__ int tile_of(const int32_t* __restrict__ plan, int E, int tile, int32_t* pairs_lds) {
    int e = 0, first = 0;
    for (; e < E; ++e) {
        const int n = plan[e + 1] - plan[e], tiles = (n + GM_ROWS - 1) / GM_ROWS;
        if (tile < tiles) {
            first = plan[e] + tile * GM_ROWS;
            break;
        }
        tile -= tiles;
    }
    if (e == E) return -1;
    for (int r = threadIdx.x; r < GM_ROWS; r += blockDim.x) pairs_lds[r] = first + r < plan[e + 1] ? plan[E + 1 + first + r] : -1;
    return e;
}

// A workgroup of four waves takes GM_ROWS pairs of one expert by GM_COLS weight rows: K goes by in
// steps of GM_BK columns that all threads stage in LDS, 16 bytes a thread and load (the pairs' rows
// gathered), in rows padded by 16 bytes so that a fragment's 32 rows spread over the banks; a wave
// takes 64 pairs by 32 weight rows.
//   HIDDEN: the weight rows are GM_COLS hidden units of gate and of up, and
//           out[pair][f] = bf16(silu(gate_f . h[pair / top]) * (up_f . h[pair / top]))
//   else:   out[pair][d] = w0_d . a[pair], float
#define GM_COLS 64
#define GM_BK 64
#define GM_LD (GM_BK + 8)
template <bool HIDDEN>
__global__ __launch_bounds__(256) void grouped_tile_kernel(const bf16_t* __restrict__ a, const int32_t* __restrict__ plan, void* __restrict__ out,
                                                           const bf16_t* __restrict__ w0, const bf16_t* __restrict__ w1, int E, int top, int K,
                                                           int N, const int32_t* __restrict__ picks, ExpertAct xa) {
    constexpr int NB = HIDDEN ? 2 : 1;
    __shared__ int32_t pairs[GM_ROWS];
    __shared__ __attribute__((aligned(16))) bf16_t As[GM_ROWS * GM_LD];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[NB * GM_COLS * GM_LD];
    const int e = tile_of(plan, E, blockIdx.x, pairs);
    if (e < 0) return;
    __syncthreads();
    const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE, l32 = lane % 32, kq = lane / 32;
    const int rh = wave / 2, uh = wave % 2, n0 = blockIdx.y * GM_COLS;
    f32x16 acc[2][NB];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;
    // what this thread stages at every step: chunk `ch` of four pairs' rows and of two (or four) weight rows
    const int ch = tid % 8, r_first = tid / 8;              // rows r_first, r_first + 32, ...
    const bf16_t* a_src[GM_ROWS / 32];
#pragma unroll
    for (int c = 0; c < GM_ROWS / 32; ++c) {
        const int pair = pairs[r_first + 32 * c];
        a_src[c] = pair >= 0 ? a + (size_t)(HIDDEN ? pair / top : pair) * K + ch * 8 : nullptr;
    }
    const bf16_t* b_src[NB * GM_COLS / 32];
#pragma unroll
    for (int c = 0; c < NB * GM_COLS / 32; ++c) {
        const int r = r_first + 32 * c;                     // rows GM_COLS and up are the second matrix's
        const bf16_t* base = r < GM_COLS ? w0 : w1;
        b_src[c] = base + ((size_t)e * N + min(n0 + r % GM_COLS, N - 1)) * K + ch * 8;
    }
    for (int k0 = 0; k0 < K; k0 += GM_BK) {
        const bool inside = k0 + ch * 8 < K;                // (K is a multiple of 16, a chunk lies inside or outside)
        bf16x8 av[GM_ROWS / 32], bv[NB * GM_COLS / 32];
#pragma unroll
        for (int c = 0; c < GM_ROWS / 32; ++c) av[c] = a_src[c] && inside ? load_chunk(a_src[c] + k0) : zero_chunk();
#pragma unroll
        for (int c = 0; c < NB * GM_COLS / 32; ++c) bv[c] = inside ? load_chunk(b_src[c] + k0) : zero_chunk();
        __syncthreads();                                    // the step before has been read
#pragma unroll
        for (int c = 0; c < GM_ROWS / 32; ++c) *(bf16x8*)(As + (r_first + 32 * c) * GM_LD + ch * 8) = av[c];
#pragma unroll
        for (int c = 0; c < NB * GM_COLS / 32; ++c) *(bf16x8*)(Bs + (r_first + 32 * c) * GM_LD + ch * 8) = bv[c];
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < GM_BK / 16; ++ks) {
            const int col = ks * 16 + kq * 8;
            const bf16x8 a0 = *(const bf16x8*)(As + (rh * 64 + l32) * GM_LD + col);
            const bf16x8 a1 = *(const bf16x8*)(As + (rh * 64 + 32 + l32) * GM_LD + col);
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const bf16x8 bj = *(const bf16x8*)(Bs + (j * GM_COLS + uh * 32 + l32) * GM_LD + col);
                acc[0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, bj, acc[0][j], 0, 0, 0);
                acc[1][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, bj, acc[1][j], 0, 0, 0);
            }
        }
    }
    const int n = n0 + uh * 32 + l32;
    if (n >= N) return;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            const int pair = pairs[rh * 64 + i * 32 + 8 * (q / 4) + q % 4 + 4 * kq];
            if (pair < 0) continue;
            if constexpr (HIDDEN) {
                const float on_input = xa.weight_on_input ? ((const float*)(picks + (size_t)(pair / top) * 2 * top + top))[pair % top] : 1.f;
                ((bf16_t*)out)[(size_t)pair * N + n] = f32_to_bf16_bits(expert_act(xa, acc[i][0][q] * on_input, acc[i][NB - 1][q] * on_input));
            } else {
                ((float*)out)[(size_t)pair * N + n] = acc[i][0][q];
            }
        }
}

// out[row] (+)= sum_k w[row][k] y[row][k], in the order of the picks
__global__ void grouped_sum_kernel(const float* __restrict__ y, const int32_t* __restrict__ picks, float* __restrict__ out, int E, int top, int D,
                                   int adds, const bf16_t* __restrict__ h, int identity, int plain_sum) {
    const size_t row = blockIdx.x;
    const int32_t* ids = picks + row * 2 * top;
    const float* w = (const float*)(ids + top);
    const float same = identity > 0 ? identity_weight(ids, w, top, E, identity) : 0.f;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        float total = 0.f;
        for (int k = 0; k < top; ++k)
            if (ids[k] >= 0 && ids[k] < E) total += (plain_sum ? 1.f : w[k]) * y[(row * top + k) * D + d];
        out[row * D + d] = (adds ? out[row * D + d] : 0.f) + total + (same != 0.f ? same * bf16_bits_to_f32(h[row * D + d]) : 0.f);
    }
}

#define GM_FROM_ROWS 64      // rows of a step from which the matrix cores take the experts

extern "C" int picolm_call_routed_experts(void* user, const picolm_step_view* v) {
    const picolm_routed_experts_args* a = (const picolm_routed_experts_args*)user;
    VIEW_REQUIRE("routed_experts", v);
    PICOLM_REQUIRE(a && a->gate && a->up && a->down && v->in && v->out && v->extra[0] && v->extra[1], "routed_experts: weights or buffers are missing");
    const int E = a->experts, top = a->top, D = a->width, F = a->ff;
    PICOLM_REQUIRE(E > 0 && top > 0 && a->identity >= 0 && top <= E + a->identity && D > 0 && F > 0 && (a->weight_dt == PICOLM_F32 || a->weight_dt == PICOLM_BF16),
                   "routed_experts: %d picks among %d experts of %d to %d", top, E, D, F);
    PICOLM_REQUIRE(v->dtype == PICOLM_BF16 || a->weight_dt == PICOLM_F32, "routed_experts: the 32-bit engine takes 32-bit weights");
    PICOLM_REQUIRE(v->in_row_bytes >= D * elem_bytes(v->dtype) && v->out_row_bytes >= D * 4 && v->extra_row_bytes[0] >= 2 * top * 4 &&
                       v->extra_row_bytes[1] >= (int64_t)top * F * 4,
                   "routed_experts: rows too short for a width of %d, %d picks and %d hidden units", D, top, F);
    PICOLM_REQUIRE(a->act == 0 || (a->act == 1 && a->limit > 0.f), "routed_experts: activation %d (limit %g) is not known", a->act, (double)a->limit);
    PICOLM_REQUIRE(!a->weight_on_input || a->identity == 0, "routed_experts: weights on the experts' input and picks that give the input back do not go together");
    const ExpertAct xa = {a->act, a->limit, a->alpha, a->weight_on_input};
    const int plain_sum = a->weight_on_input ? 1 : 0;
    const size_t lds_a = sizeof(float) * (size_t)D, lds_b = sizeof(float) * (size_t)top * F;
    PICOLM_REQUIRE(lds_a <= 64 * 1024 && lds_b <= 64 * 1024, "routed_experts: a width of %d or %d picks of %d hidden units exceed 64 KiB of LDS", D,
                   top, F);
    PICOLM_REQUIRE(ceil_div(F, MOE_UNITS) <= 65535 && ceil_div(D, MOE_UNITS) <= 65535 && (int64_t)v->rows * top < (1ll << 31),
                   "routed_experts: the sizes exceed the grid");
    if (v->rows <= 0) return 0;
    const int32_t* picks = (const int32_t*)v->extra[0];
    float* act = (float*)v->extra[1];
    if (v->dtype == PICOLM_BF16 && a->weight_dt == PICOLM_BF16 && v->rows >= GM_FROM_ROWS && D % 16 == 0 && F % 16 == 0 && E <= GM_MAX_EXPERTS &&
        v->extra[2] && v->extra[3]) {
        const int64_t n_pairs = (int64_t)v->rows * top;
        PICOLM_REQUIRE(v->extra_row_bytes[2] >= (int64_t)top * D * 4 && v->extra_row_bytes[3] >= (int64_t)(top + E + 1) * 4,
                       "routed_experts: scratch rows too short for the sorted pairs or their outputs");
        int32_t* plan = (int32_t*)v->extra[3];
        float* y = (float*)v->extra[2];
        moe_plan_kernel<<<1, 1024, sizeof(int32_t) * (2 * (size_t)E + 1), v->stream>>>(picks, plan, E, top, (int)n_pairs);
        PICOLM_LAUNCH_CHECK("routed_experts (plan)");
        const unsigned tiles = (unsigned)(ceil_div64(n_pairs, GM_ROWS) + E);      // no more than these are filled; the rest leave at once
        grouped_tile_kernel<true><<<dim3(tiles, ceil_div(F, GM_COLS)), 256, 0, v->stream>>>((const bf16_t*)v->in, plan, act, (const bf16_t*)a->gate,
                                                                                           (const bf16_t*)a->up, E, top, D, F, picks, xa);
        PICOLM_LAUNCH_CHECK("routed_experts (hidden, grouped)");
        grouped_tile_kernel<false><<<dim3(tiles, ceil_div(D, GM_COLS)), 256, 0, v->stream>>>((const bf16_t*)act, plan, y, (const bf16_t*)a->down,
                                                                                            nullptr, E, top, F, D, picks, xa);
        PICOLM_LAUNCH_CHECK("routed_experts (down, grouped)");
        grouped_sum_kernel<<<v->rows, 256, 0, v->stream>>>(y, picks, (float*)v->out, E, top, D, a->adds, (const bf16_t*)v->in, a->identity, plain_sum);
        PICOLM_LAUNCH_CHECK("routed_experts (sum)");
        return 0;
    }
    const dim3 grid_a((unsigned)(v->rows * top), ceil_div(F, MOE_UNITS)), grid_b(v->rows, ceil_div(D, MOE_UNITS));
    if (a->weight_dt == PICOLM_F32 && v->dtype == PICOLM_F32) {
        expert_hidden_kernel<float, float><<<grid_a, 256, lds_a, v->stream>>>((const float*)v->in, picks, act, (const float*)a->gate,
                                                                              (const float*)a->up, E, top, D, F, xa);
        PICOLM_LAUNCH_CHECK("routed_experts (hidden)");
        expert_down_kernel<float, float><<<grid_b, 256, lds_b, v->stream>>>(act, picks, (float*)v->out, (const float*)a->down, E, top, D, F, a->adds,
                                                                            (const float*)v->in, a->identity, plain_sum);
    } else if (a->weight_dt == PICOLM_F32) {
        expert_hidden_kernel<float, bf16_t><<<grid_a, 256, lds_a, v->stream>>>((const bf16_t*)v->in, picks, act, (const float*)a->gate,
                                                                               (const float*)a->up, E, top, D, F, xa);
        PICOLM_LAUNCH_CHECK("routed_experts (hidden)");
        expert_down_kernel<float, bf16_t><<<grid_b, 256, lds_b, v->stream>>>(act, picks, (float*)v->out, (const float*)a->down, E, top, D, F, a->adds,
                                                                             (const bf16_t*)v->in, a->identity, plain_sum);
    } else {
        expert_hidden_kernel<bf16_t, bf16_t><<<grid_a, 256, lds_a, v->stream>>>((const bf16_t*)v->in, picks, act, (const bf16_t*)a->gate,
                                                                                (const bf16_t*)a->up, E, top, D, F, xa);
        PICOLM_LAUNCH_CHECK("routed_experts (hidden)");
        expert_down_kernel<bf16_t, bf16_t><<<grid_b, 256, lds_b, v->stream>>>(act, picks, (float*)v->out, (const bf16_t*)a->down, E, top, D, F, a->adds,
                                                                              (const bf16_t*)v->in, a->identity, plain_sum);
    }
    PICOLM_LAUNCH_CHECK("routed_experts (down)");
    return 0;
}
