// Called operations of the library's own (mixers.h) that work row by row: positions added to the
// embedding, the blend of a token with the one before it, gates, norms of a stretch of columns, a
// product per head, and the sum-then-norm of layers that norm after adding.  Every function checks
// what it is handed on the host, then queues its kernels on the step's stream; what they do
// depends on device memory only, so a decode step that holds them can be recorded and replayed.
//
// All arithmetic is float (angles double); rows that feed a product are written in the engine's dtype.
#include "mixers.h"

#include "api.h"
#include "common.h"
#include "gemm_mfma.h"

#define VIEW_REQUIRE(who, v)                                                                                      \
    PICOLM_REQUIRE((v) && (v)->struct_bytes == (int32_t)sizeof(picolm_step_view), "%s: the step view is of another version", who)

static inline int elem_bytes(int dt) { return dt == PICOLM_F32 ? 4 : 2; }
static inline bool known_dtype(int dt) { return dt == PICOLM_F32 || dt == PICOLM_BF16; }

__device__ __forceinline__ float silu_f(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }

// an element of a buffer whose dtype is known at run time
__device__ __forceinline__ float load_as_f32(const void* p, size_t i, int dt) {
    return dt == PICOLM_F32 ? ((const float*)p)[i] : bf16_bits_to_f32(((const bf16_t*)p)[i]);
}
__device__ __forceinline__ void store_from_f32(void* p, size_t i, int dt, float v) {
    if (dt == PICOLM_F32) ((float*)p)[i] = v;
    else ((bf16_t*)p)[i] = f32_to_bf16_bits(v);
}

// ---- positions ------------------------------------------------------------------------------------
__global__ void add_positions_kernel(float* __restrict__ x, const int32_t* __restrict__ tok_pos, const double* __restrict__ freq, int W) {
    const size_t row = blockIdx.x;
    const double p = (double)tok_pos[row];
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const double angle = p * freq[c >> 1];
        x[row * W + c] += (float)((c & 1) ? cos(angle) : sin(angle));
    }
}

extern "C" int picolm_call_add_positions(void* user, const picolm_step_view* v) {
    const picolm_add_positions_args* a = (const picolm_add_positions_args*)user;
    VIEW_REQUIRE("add_positions", v);
    PICOLM_REQUIRE(a && a->freq && a->width > 0 && v->out && v->tok_pos, "add_positions: the table or the rows are missing");
    PICOLM_REQUIRE(v->out_row_bytes >= a->width * 4, "add_positions: rows too short for a width of %d", a->width);
    if (v->rows <= 0) return 0;
    add_positions_kernel<<<v->rows, 256, 0, v->stream>>>((float*)v->out, v->tok_pos, a->freq, a->width);
    PICOLM_LAUNCH_CHECK("add_positions");
    return 0;
}

// ---- a token blended with the one before it ---------------------------------------------------------
// One workgroup a row.  A sequence that brings one token reads its state and then writes it in the
// same thread; the state of a sequence that brings more is written by the kernel after this one.
template <typename T>
__global__ void token_shift_kernel(const float* __restrict__ x, T* __restrict__ y, T* __restrict__ plain, float* __restrict__ state,
                                   int64_t slot_floats, const float* __restrict__ mu, int W, const int32_t* __restrict__ tok_seq,
                                   const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_slot) {
    const int row = blockIdx.x;
    const int seq = tok_seq[row], first = cu_seqlens[seq], n = cu_seqlens[seq + 1] - first;
    float* st = state + (size_t)seq_slot[seq] * slot_floats;
    const float* prev = row > first ? x + (size_t)(row - 1) * W : st;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float xv = x[(size_t)row * W + c], pv = prev[c];
        y[(size_t)row * W + c] = from_f32<T>(xv + (pv - xv) * mu[c]);
        if (plain) plain[(size_t)row * W + c] = from_f32<T>(xv);
        if (n == 1) st[c] = xv;
    }
}

__global__ void token_shift_state_kernel(const float* __restrict__ x, float* __restrict__ state, int64_t slot_floats, int W,
                                         const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_slot) {
    const int seq = blockIdx.x;
    const int first = cu_seqlens[seq], n = cu_seqlens[seq + 1] - first;
    if (n <= 1) return;
    float* st = state + (size_t)seq_slot[seq] * slot_floats;
    for (int c = threadIdx.x; c < W; c += blockDim.x) st[c] = x[(size_t)(first + n - 1) * W + c];
}

extern "C" int picolm_call_token_shift(void* user, const picolm_step_view* v) {
    const picolm_token_shift_args* a = (const picolm_token_shift_args*)user;
    VIEW_REQUIRE("token_shift", v);
    PICOLM_REQUIRE(a && a->mu && a->width > 0 && v->in && v->out && v->state, "token_shift: weights, buffers or state are missing");
    const int es = elem_bytes(v->dtype), W = a->width;
    PICOLM_REQUIRE(v->in_row_bytes >= W * 4 && v->out_row_bytes >= W * es && (!v->extra[0] || v->extra_row_bytes[0] >= W * es),
                   "token_shift: rows too short for a width of %d", W);
    PICOLM_REQUIRE(a->state_off >= 0 && (a->state_off + W) * 4 <= v->state_bytes_per_slot,
                   "token_shift: the state of a slot has %lld bytes, a row at %lld needs %lld", (long long)v->state_bytes_per_slot,
                   (long long)a->state_off, (long long)((a->state_off + W) * 4));
    if (v->n_tokens <= 0) return 0;
    const int64_t slot_floats = v->state_bytes_per_slot / 4;
    float* state = (float*)v->state + a->state_off;
    if (v->dtype == PICOLM_F32)
        token_shift_kernel<float><<<v->n_tokens, 256, 0, v->stream>>>((const float*)v->in, (float*)v->out, (float*)v->extra[0], state, slot_floats,
                                                                     a->mu, W, v->tok_seq, v->cu_seqlens, v->seq_slot);
    else
        token_shift_kernel<bf16_t><<<v->n_tokens, 256, 0, v->stream>>>((const float*)v->in, (bf16_t*)v->out, (bf16_t*)v->extra[0], state,
                                                                      slot_floats, a->mu, W, v->tok_seq, v->cu_seqlens, v->seq_slot);
    PICOLM_LAUNCH_CHECK("token_shift");
    if (!v->is_decode) {
        token_shift_state_kernel<<<v->n_seq, 256, 0, v->stream>>>((const float*)v->in, state, slot_floats, W, v->cu_seqlens, v->seq_slot);
        PICOLM_LAUNCH_CHECK("token_shift (state)");
    }
    return 0;
}

// ---- a gate over columns ---------------------------------------------------------------------------
__global__ void gate_rows_kernel(const void* __restrict__ x, int x_stride, int x_off, int x_dt, const float* __restrict__ g, int g_stride,
                                 int g_off, const float* __restrict__ bias, void* __restrict__ out, int out_dt, int W, int act, int64_t n, int g_per_row) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const size_t row = i / W;
        const int c = (int)(i % W);
        float y = load_as_f32(x, row * x_stride + x_off + c, x_dt);
        if (act) {
            const float z = g_per_row ? g[row * g_stride + g_off] : g[row * g_stride + g_off + c] + (bias ? bias[c] : 0.f);
            y *= act == 1 ? silu_f(z) : sigmoid_f(z);
        }
        store_from_f32(out, (size_t)i, out_dt, y);
    }
}

extern "C" int picolm_call_gate_rows(void* user, const picolm_step_view* v) {
    const picolm_gate_rows_args* a = (const picolm_gate_rows_args*)user;
    VIEW_REQUIRE("gate_rows", v);
    PICOLM_REQUIRE(a && v->in && v->out && a->width > 0 && a->act >= 0 && a->act <= 2 && known_dtype(a->x_dtype) && known_dtype(a->out_dtype),
                   "gate_rows: buffers are missing, or an unknown gate or dtype");
    PICOLM_REQUIRE(a->x_off >= 0 && a->x_off + a->width <= a->x_stride && v->in_row_bytes >= a->x_stride * elem_bytes(a->x_dtype) &&
                       v->out_row_bytes >= a->width * elem_bytes(a->out_dtype),
                   "gate_rows: rows too short for %d columns at %d of %d", a->width, a->x_off, a->x_stride);
    PICOLM_REQUIRE(!a->act || (v->extra[0] && a->g_off >= 0 && a->g_off + (a->g_per_row ? 1 : a->width) <= a->g_stride &&
                               v->extra_row_bytes[0] >= a->g_stride * 4 && !(a->g_per_row && a->bias)),
                   "gate_rows: the gate's rows of %d floats do not hold %d at %d", a->g_stride, a->width, a->g_off);
    if (v->rows <= 0) return 0;
    const int64_t n = (int64_t)v->rows * a->width;
    const unsigned blocks = (unsigned)std::min<int64_t>(ceil_div64(n, 256), 65536);
    gate_rows_kernel<<<blocks, 256, 0, v->stream>>>(v->in, a->x_stride, a->x_off, a->x_dtype, (const float*)v->extra[0], a->g_stride, a->g_off,
                                                   a->bias, v->out, a->out_dtype, a->width, a->act, n, a->g_per_row);
    PICOLM_LAUNCH_CHECK("gate_rows");
    return 0;
}

// ---- the norm of a stretch of columns ------------------------------------------------------------------
__global__ __launch_bounds__(1024) void slice_norm_kernel(const float* __restrict__ x, int in_stride, int in_off, void* __restrict__ out,
                                                         int out_stride, int out_off, int out_dt, const float* __restrict__ weight, int W,
                                                         float eps) {
    __shared__ float scratch[16];
    const size_t row = blockIdx.x;
    const float* xr = x + row * in_stride + in_off;
    float ssq = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) ssq += xr[c] * xr[c];
    ssq = block_sum(ssq, scratch);
    const float inv = 1.f / sqrtf(ssq / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += blockDim.x) store_from_f32(out, row * out_stride + out_off + c, out_dt, xr[c] * inv * weight[c]);
}

extern "C" int picolm_call_slice_norm(void* user, const picolm_step_view* v) {
    const picolm_slice_norm_args* a = (const picolm_slice_norm_args*)user;
    VIEW_REQUIRE("slice_norm", v);
    PICOLM_REQUIRE(a && a->weight && v->in && v->out && a->width > 0 && known_dtype(a->out_dtype), "slice_norm: weights or buffers are missing");
    PICOLM_REQUIRE(a->in_off >= 0 && a->in_off + a->width <= a->in_stride && v->in_row_bytes >= a->in_stride * 4 && a->out_off >= 0 &&
                       a->out_off + a->width <= a->out_stride && v->out_row_bytes >= a->out_stride * elem_bytes(a->out_dtype),
                   "slice_norm: rows too short for %d columns at the offsets named", a->width);
    PICOLM_REQUIRE(v->in != v->out, "slice_norm: input and output differ");
    if (v->rows <= 0) return 0;
    slice_norm_kernel<<<v->rows, a->width >= 2048 ? 1024 : 256, 0, v->stream>>>((const float*)v->in, a->in_stride, a->in_off, v->out, a->out_stride,
                                                                               a->out_off, a->out_dtype, a->weight, a->width, a->eps);
    PICOLM_LAUNCH_CHECK("slice_norm");
    return 0;
}

// ---- a product per head -----------------------------------------------------------------------------
// One workgroup per (HL_ROWS rows, head, HL_COLS outputs): the rows' inputs wait in LDS as floats and
// every weight that is read meets all of them.  Not transposed: a wave takes four outputs at a
// time, its lanes along the input (adjacent lanes read adjacent weights).  Transposed: a thread per
// output and quarter of the input, adjacent threads read adjacent weights, and the quarters meet in
// LDS.  Either way a thread has several loads on their way at once: a decode step has few
// workgroups, and what they wait for is the latency of their loads.
#define HL_ROWS 8
#define HL_COLS 64
template <typename TW>
__global__ __launch_bounds__(256) void head_linear_kernel(picolm_head_linear_args a, const void* __restrict__ in, void* __restrict__ out,
                                                          const float* __restrict__ gate, int n_rows, int cols) {
    extern __shared__ float hl_in[];      // [HL_ROWS][in_dim] | partial sums [4][HL_ROWS][HL_COLS] (transposed)
    const int head = blockIdx.y, row0 = blockIdx.x * HL_ROWS, nr = min(HL_ROWS, n_rows - row0);
    const int K = a.in_dim, N = a.out_dim, o0 = blockIdx.z * cols;       // (cols is HL_COLS when transposed)
    const size_t in_head = (size_t)head * (a.in_head_stride ? a.in_head_stride : K), out_head = (size_t)head * (a.out_head_stride ? a.out_head_stride : N);
    for (int idx = threadIdx.x; idx < HL_ROWS * K; idx += blockDim.x) {
        const int r = idx / K, i = idx % K;
        hl_in[idx] = r < nr ? load_as_f32(in, (size_t)(row0 + r) * a.in_stride + a.in_off + in_head + i, a.in_dtype) : 0.f;
    }
    __syncthreads();
    const TW* w = (const TW*)a.weight;
    auto finish = [&](int r, int o, float acc) {
        const size_t row = row0 + r;
        if (a.gate_act) {
            const float z = gate[row * a.gate_stride + a.gate_off + (a.gate_per_head ? (size_t)head : (size_t)head * N + o)];
            acc *= a.gate_act == 1 ? silu_f(z) : sigmoid_f(z);
        }
        store_from_f32(out, row * a.out_stride + a.out_off + out_head + o, a.out_dtype, acc);
    };
    if (a.transposed) {
        float* part = hl_in + HL_ROWS * K;
        const TW* wh = w + (size_t)head * K * N;
        const int col = threadIdx.x % HL_COLS, quarter = threadIdx.x / HL_COLS, o = o0 + col;
        const int per = (K + 3) / 4, i0 = quarter * per, i1 = min(K, i0 + per);
        float acc[HL_ROWS];
#pragma unroll
        for (int r = 0; r < HL_ROWS; ++r) acc[r] = 0.f;
        if (o < N) {
#pragma unroll 8
            for (int i = i0; i < i1; ++i) {
                const float wv = to_f32<TW>(wh[(size_t)i * N + o]);
#pragma unroll
                for (int r = 0; r < HL_ROWS; ++r) acc[r] += wv * hl_in[r * K + i];
            }
        }
#pragma unroll
        for (int r = 0; r < HL_ROWS; ++r) part[(quarter * HL_ROWS + r) * HL_COLS + col] = acc[r];
        __syncthreads();
        for (int idx = threadIdx.x; idx < HL_ROWS * HL_COLS; idx += blockDim.x) {
            const int r = idx / HL_COLS, c = idx % HL_COLS;
            if (r < nr && o0 + c < N)
                finish(r, o0 + c, part[(0 * HL_ROWS + r) * HL_COLS + c] + part[(1 * HL_ROWS + r) * HL_COLS + c] +
                                      part[(2 * HL_ROWS + r) * HL_COLS + c] + part[(3 * HL_ROWS + r) * HL_COLS + c]);
        }
    } else {
        const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
        const TW* wh = w + (size_t)head * N * K;
        const int o_end = min(N, o0 + cols);
        for (int ob = o0 + wave * 4; ob < o_end; ob += 16) {        // four waves, four outputs each at a time
            float acc[4][HL_ROWS];
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int r = 0; r < HL_ROWS; ++r) acc[u][r] = 0.f;
            for (int i = lane; i < K; i += WAVE) {
                float wv[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) wv[u] = ob + u < o_end ? to_f32<TW>(wh[(size_t)(ob + u) * K + i]) : 0.f;
#pragma unroll
                for (int r = 0; r < HL_ROWS; ++r) {
                    const float x = hl_in[r * K + i];
#pragma unroll
                    for (int u = 0; u < 4; ++u) acc[u][r] += wv[u] * x;
                }
            }
            float mine = 0.f;                      // lane 8 u + r takes the sum of output u and row r: the gates are then loaded side by side
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int r = 0; r < HL_ROWS; ++r) {
                    const float s = wave_sum(acc[u][r]);
                    if (lane == u * HL_ROWS + r) mine = s;
                }
            const int u = lane / HL_ROWS, r = lane % HL_ROWS;
            if (lane < 4 * HL_ROWS && r < nr && ob + u < o_end) finish(r, ob + u, mine);
        }
    }
}

// The same on the matrix cores, for steps of many rows in bfloat16 (not transposed): a wave takes 32
// rows by 32 outputs of a head with v_mfma_f32_32x32x16_bf16, its operands straight from global
// memory (float inputs are rounded to bfloat16 on the way, as every product's input is).
__global__ __launch_bounds__(256) void head_linear_mfma_kernel(picolm_head_linear_args a, const void* __restrict__ in, void* __restrict__ out,
                                                               const float* __restrict__ gate, int n_rows) {
    const int head = blockIdx.y, row0 = blockIdx.x * 32, K = a.in_dim, N = a.out_dim;
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, l32 = lane % 32, kq = lane / 32;
    const int n0 = (blockIdx.z * 4 + wave) * 32;
    if (n0 >= N) return;
    const int my_row = row0 + l32;
    const size_t in_at = (size_t)min(my_row, n_rows - 1) * a.in_stride + a.in_off + (size_t)head * (a.in_head_stride ? a.in_head_stride : K) + kq * 8;
    const size_t out_head = (size_t)head * (a.out_head_stride ? a.out_head_stride : N);
    const bf16_t* w_row = (const bf16_t*)a.weight + ((size_t)head * N + min(n0 + l32, N - 1)) * K + kq * 8;
    f32x16 acc;
#pragma unroll
    for (int q = 0; q < 16; ++q) acc[q] = 0.f;
#pragma unroll 4
    for (int k = 0; k < K; k += 16) {
        bf16x8 av;
        if (a.in_dtype == PICOLM_F32) {
            const float4 lo = *(const float4*)((const float*)in + in_at + k), hi = *(const float4*)((const float*)in + in_at + k + 4);
            const float f[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            bf16_t* bits = (bf16_t*)&av;
#pragma unroll
            for (int i = 0; i < 8; ++i) bits[i] = f32_to_bf16_bits(f[i]);
        } else {
            av = load_chunk((const bf16_t*)in + in_at + k);
        }
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, load_chunk(w_row + k), acc, 0, 0, 0);
    }
    const int o = n0 + l32;
    if (o >= N) return;
#pragma unroll
    for (int q = 0; q < 16; ++q) {
        const size_t row = row0 + 8 * (q / 4) + q % 4 + 4 * kq;
        if (row >= (size_t)n_rows) continue;
        float y = acc[q];
        if (a.gate_act) {
            const float z = gate[row * a.gate_stride + a.gate_off + (a.gate_per_head ? (size_t)head : (size_t)head * N + o)];
            y *= a.gate_act == 1 ? silu_f(z) : sigmoid_f(z);
        }
        store_from_f32(out, row * a.out_stride + a.out_off + out_head + o, a.out_dtype, y);
    }
}
#define HL_MFMA_FROM_ROWS 32

extern "C" int picolm_call_head_linear(void* user, const picolm_step_view* v) {
    const picolm_head_linear_args* a = (const picolm_head_linear_args*)user;
    VIEW_REQUIRE("head_linear", v);
    PICOLM_REQUIRE(a && a->weight && v->in && v->out && v->in != v->out, "head_linear: weights or buffers are missing (input and output differ)");
    PICOLM_REQUIRE(a->heads > 0 && a->heads <= 65535 && a->in_dim > 0 && a->out_dim > 0 && known_dtype(a->weight_dt) && known_dtype(a->in_dtype) &&
                       known_dtype(a->out_dtype) && a->gate_act >= 0 && a->gate_act <= 2,
                   "head_linear: %d heads of %d to %d, or an unknown dtype or gate", a->heads, a->in_dim, a->out_dim);
    const int64_t in_hs = a->in_head_stride ? a->in_head_stride : a->in_dim, out_hs = a->out_head_stride ? a->out_head_stride : a->out_dim;
    PICOLM_REQUIRE(in_hs >= a->in_dim && out_hs >= a->out_dim, "head_linear: heads %lld and %lld apart overlap at sizes of %d and %d", (long long)in_hs,
                   (long long)out_hs, a->in_dim, a->out_dim);
    PICOLM_REQUIRE(a->in_off >= 0 && a->in_off + (a->heads - 1) * in_hs + a->in_dim <= a->in_stride &&
                       v->in_row_bytes >= (int64_t)a->in_stride * elem_bytes(a->in_dtype) && a->out_off >= 0 &&
                       a->out_off + (a->heads - 1) * out_hs + a->out_dim <= a->out_stride &&
                       v->out_row_bytes >= (int64_t)a->out_stride * elem_bytes(a->out_dtype),
                   "head_linear: rows too short for %d heads at the offsets named", a->heads);
    PICOLM_REQUIRE(!a->gate_act || (v->extra[0] && a->gate_off >= 0 &&
                                    a->gate_off + (int64_t)a->heads * (a->gate_per_head ? 1 : a->out_dim) <= a->gate_stride &&
                                    v->extra_row_bytes[0] >= (int64_t)a->gate_stride * 4),
                   "head_linear: the gate's rows of %d floats do not hold the heads at %d", a->gate_stride, a->gate_off);
    const size_t lds = sizeof(float) * (HL_ROWS * (size_t)a->in_dim + (a->transposed ? 4 * HL_ROWS * HL_COLS : 0));
    PICOLM_REQUIRE(lds <= 64 * 1024 && ceil_div(a->out_dim, HL_COLS) <= 65535, "head_linear: an input of %d a head needs %zu bytes of LDS",
                   a->in_dim, lds);
    if (v->rows <= 0) return 0;
    if (v->dtype == PICOLM_BF16 && a->weight_dt == PICOLM_BF16 && !a->transposed && v->rows >= HL_MFMA_FROM_ROWS && a->in_dim % 16 == 0 &&
        a->in_off % 8 == 0 && a->in_stride % 8 == 0 && in_hs % 8 == 0 && ceil_div(a->out_dim, 128) <= 65535) {
        head_linear_mfma_kernel<<<dim3(ceil_div(v->rows, 32), a->heads, ceil_div(a->out_dim, 128)), 256, 0, v->stream>>>(
            *a, v->in, v->out, (const float*)v->extra[0], v->rows);
        PICOLM_LAUNCH_CHECK("head_linear (matrix cores)");
        return 0;
    }
    // a step of few rows has few workgroups, each with a chain of loads and sums in a row: not transposed, a workgroup
    // then takes 16 outputs (its four waves four each, once) instead of 64
    const int row_groups = ceil_div(v->rows, HL_ROWS);
    const int cols = !a->transposed && (int64_t)row_groups * a->heads * ceil_div(a->out_dim, HL_COLS) < 256 && ceil_div(a->out_dim, 16) <= 65535 ? 16 : HL_COLS;
    const dim3 grid(row_groups, a->heads, ceil_div(a->out_dim, cols));
    if (a->weight_dt == PICOLM_F32)
        head_linear_kernel<float><<<grid, 256, lds, v->stream>>>(*a, v->in, v->out, (const float*)v->extra[0], v->rows, cols);
    else
        head_linear_kernel<bf16_t><<<grid, 256, lds, v->stream>>>(*a, v->in, v->out, (const float*)v->extra[0], v->rows, cols);
    PICOLM_LAUNCH_CHECK("head_linear");
    return 0;
}

// ---- the sum and the norm of a layer that norms after adding ---------------------------------------------
template <typename T>
__global__ __launch_bounds__(1024) void gated_postnorm_kernel(float* __restrict__ x, const float* __restrict__ u, const float* __restrict__ g,
                                                             const float* __restrict__ bias, const float* __restrict__ weight, int W,
                                                             float alpha, float eps, T* __restrict__ plain) {
    __shared__ float scratch[16];
    const size_t row = blockIdx.x;
    float* xr = x + row * W;
    const float* ur = u + row * W;
    const float* gr = g ? g + row * W : nullptr;
    auto sum_at = [&](int c) {
        float uv = ur[c];
        if (gr) uv *= sigmoid_f(gr[c] + (bias ? bias[c] : 0.f));
        return alpha * xr[c] + uv;
    };
    float ssq = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float s = sum_at(c);
        ssq += s * s;
    }
    ssq = block_sum(ssq, scratch);
    const float inv = 1.f / sqrtf(ssq / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float y = sum_at(c) * inv * weight[c];
        xr[c] = y;                                                 // a thread writes what only it reads
        if (plain) plain[row * W + c] = from_f32<T>(y);
    }
}

extern "C" int picolm_call_gated_postnorm(void* user, const picolm_step_view* v) {
    const picolm_gated_postnorm_args* a = (const picolm_gated_postnorm_args*)user;
    VIEW_REQUIRE("gated_postnorm", v);
    PICOLM_REQUIRE(a && a->weight && v->in && v->out && a->width > 0, "gated_postnorm: weights or buffers are missing");
    PICOLM_REQUIRE(v->in_row_bytes >= a->width * 4 && v->out_row_bytes >= a->width * 4 && (!v->extra[0] || v->extra_row_bytes[0] >= a->width * 4) &&
                       (!v->extra[1] || v->extra_row_bytes[1] >= a->width * elem_bytes(v->dtype)),
                   "gated_postnorm: rows too short for a width of %d", a->width);
    if (v->rows <= 0) return 0;
    const int threads = a->width >= 2048 ? 1024 : 256;
    if (v->dtype == PICOLM_F32)
        gated_postnorm_kernel<float><<<v->rows, threads, 0, v->stream>>>((float*)v->out, (const float*)v->in, (const float*)v->extra[0], a->gate_bias,
                                                                        a->weight, a->width, a->alpha, a->eps, (float*)v->extra[1]);
    else
        gated_postnorm_kernel<bf16_t><<<v->rows, threads, 0, v->stream>>>((float*)v->out, (const float*)v->in, (const float*)v->extra[0], a->gate_bias,
                                                                         a->weight, a->width, a->alpha, a->eps, (bf16_t*)v->extra[1]);
    PICOLM_LAUNCH_CHECK("gated_postnorm");
    return 0;
}

// ---- what a forget gate per key channel gives a token --------------------------------------------------
__global__ void forget_gates_kernel(const float* __restrict__ in, int in_stride, int q_off, int f_off, float* __restrict__ out,
                                    const float* __restrict__ lower, const float* __restrict__ bias, int C, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const size_t row = i / C;
        const int c = (int)(i % C);
        const float* r = in + row * in_stride;
        const float lo = lower[c];
        const float a = lo + (1.f - lo) * sigmoid_f(r[f_off + c] + (bias ? bias[c] : 0.f));
        float* o = out + row * 3 * C;
        o[c] = silu_f(r[q_off + c]);
        o[C + c] = 1.f - a;
        o[2 * C + c] = a;
    }
}

extern "C" int picolm_call_forget_gates(void* user, const picolm_step_view* v) {
    const picolm_forget_gates_args* a = (const picolm_forget_gates_args*)user;
    VIEW_REQUIRE("forget_gates", v);
    PICOLM_REQUIRE(a && a->lower && v->in && v->out && v->in != v->out && a->channels > 0, "forget_gates: bounds or buffers are missing");
    PICOLM_REQUIRE(a->q_off >= 0 && a->q_off + a->channels <= a->in_stride && a->f_off >= 0 && a->f_off + a->channels <= a->in_stride &&
                       v->in_row_bytes >= a->in_stride * 4 && v->out_row_bytes >= (int64_t)3 * a->channels * 4,
                   "forget_gates: rows too short for %d channels at the offsets named", a->channels);
    if (v->rows <= 0) return 0;
    const int64_t n = (int64_t)v->rows * a->channels;
    const unsigned blocks = (unsigned)std::min<int64_t>(ceil_div64(n, 256), 65536);
    forget_gates_kernel<<<blocks, 256, 0, v->stream>>>((const float*)v->in, a->in_stride, a->q_off, a->f_off, (float*)v->out, a->lower, a->bias,
                                                      a->channels, n);
    PICOLM_LAUNCH_CHECK("forget_gates");
    return 0;
}

// ---- layer norm ---------------------------------------------------------------------------------------
// One workgroup a row, two passes over the row in float: the mean, then the mean of the squared
// deviations from it (not E[x^2] - mean^2, which loses the small variance of a row with a large mean).
__global__ __launch_bounds__(1024) void layer_norm_kernel(const float* __restrict__ x, size_t x_stride, const int32_t* __restrict__ gather,
                                                         void* __restrict__ out, size_t out_stride, int out_dt,
                                                         const float* __restrict__ weight, const float* __restrict__ bias, int W, float eps) {
    __shared__ float scratch[16];
    const size_t row = blockIdx.x;
    const float* xr = x + (gather ? (size_t)gather[row] : row) * x_stride;
    float sum = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) sum += xr[c];
    const float mean = block_sum(sum, scratch) / (float)W;
    __syncthreads();                                   // (the scratch is read before it is written again)
    float ssq = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float dev = xr[c] - mean;
        ssq += dev * dev;
    }
    const float inv = 1.f / sqrtf(block_sum(ssq, scratch) / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += blockDim.x)
        store_from_f32(out, row * out_stride + c, out_dt, (xr[c] - mean) * inv * weight[c] + (bias ? bias[c] : 0.f));
}

extern "C" int picolm_call_layer_norm(void* user, const picolm_step_view* v) {
    const picolm_layer_norm_args* a = (const picolm_layer_norm_args*)user;
    VIEW_REQUIRE("layer_norm", v);
    PICOLM_REQUIRE(a && a->weight && v->in && v->out && v->in != v->out && a->width > 0 && known_dtype(a->out_dtype) && a->eps > 0.f,
                   "layer_norm: weights or buffers are missing");
    PICOLM_REQUIRE(v->in_row_bytes >= a->width * 4 && v->out_row_bytes >= a->width * elem_bytes(a->out_dtype),
                   "layer_norm: rows too short for a width of %d", a->width);
    PICOLM_REQUIRE(!a->gathers || v->want_rows, "layer_norm: the step names no wanted rows");
    if (v->rows <= 0) return 0;
    layer_norm_kernel<<<v->rows, a->width >= 2048 ? 1024 : 256, 0, v->stream>>>(
        (const float*)v->in, (size_t)a->width, a->gathers ? v->want_rows : nullptr, v->out, (size_t)a->width, a->out_dtype, a->weight, a->bias,
        a->width, a->eps);
    PICOLM_LAUNCH_CHECK("layer_norm");
    return 0;
}

// ---- rotation of stretches of a row by the token's position ---------------------------------------------
// A thread a pair (or an entry that is only copied); a workgroup a row.  The stretches of the second group follow
// those of the first in the threads' order; the normed stretch comes last and takes the whole workgroup's sum.
__global__ __launch_bounds__(256) void rotate_heads_kernel(picolm_rotate_heads_args a, const float* __restrict__ in, float* __restrict__ out,
                                                           const int32_t* __restrict__ tok_pos) {
    __shared__ float scratch[16];
    const size_t row = blockIdx.x;
    const int pairs = a.dims / 2, rest = a.width - a.dims, per_head = pairs + rest;
    const int p = min(tok_pos[row], a.table_positions - 1);        // (the host has checked the step's positions against the table)
    const float* cs = a.cos_table + (size_t)p * pairs;
    const float* sn = a.sin_table + (size_t)p * pairs;
    for (int idx = threadIdx.x; idx < (a.heads + a.more_heads) * per_head; idx += blockDim.x) {
        const int head = idx / per_head, j = idx % per_head;
        const bool first = head < a.heads;
        const float* x = in + row * a.in_stride + (first ? a.in_off + (size_t)head * a.in_head_stride
                                                         : a.more_in_off + (size_t)(head - a.heads) * a.more_in_head_stride);
        float* y = out + row * a.out_stride + (first ? a.out_off + (size_t)head * a.out_head_stride
                                                     : a.more_out_off + (size_t)(head - a.heads) * a.more_out_head_stride);
        if (j < pairs) {
            const int iu = a.half ? j : 2 * j, iv = a.half ? j + pairs : 2 * j + 1;
            const float u = x[iu], w = x[iv], c = cs[j], s = sn[j];
            y[iu] = u * c - w * s;
            y[iv] = w * c + u * s;
        } else {
            y[a.dims + j - pairs] = x[a.dims + j - pairs];
        }
    }
    if (!a.norm_weight) return;                    // (the same for every thread of the grid)
    const float* xr = in + row * a.in_stride + a.norm_in_off;
    float ssq = 0.f;
    for (int c = threadIdx.x; c < a.norm_width; c += blockDim.x) ssq += xr[c] * xr[c];
    ssq = block_sum(ssq, scratch);
    const float inv = 1.f / sqrtf(ssq / (float)a.norm_width + a.norm_eps);
    for (int c = threadIdx.x; c < a.norm_width; c += blockDim.x) out[row * a.out_stride + a.norm_out_off + c] = xr[c] * inv * a.norm_weight[c];
}

extern "C" int picolm_call_rotate_heads(void* user, const picolm_step_view* v) {
    const picolm_rotate_heads_args* a = (const picolm_rotate_heads_args*)user;
    VIEW_REQUIRE("rotate_heads", v);
    PICOLM_REQUIRE(a && a->cos_table && a->sin_table && v->in && v->out && v->tok_pos && v->rows == v->n_tokens,
                   "rotate_heads: tables or buffers are missing (it covers the step's rows)");
    PICOLM_REQUIRE(a->dims > 0 && a->dims % 2 == 0 && a->width >= a->dims && a->heads > 0 && a->table_positions > 0 &&
                       a->in_head_stride >= (a->heads > 1 ? a->width : 0) && a->out_head_stride >= (a->heads > 1 ? a->width : 0),
                   "rotate_heads: %d stretches of %d entries of which %d turn", a->heads, a->width, a->dims);
    PICOLM_REQUIRE(a->in_off >= 0 && a->in_off + (int64_t)(a->heads - 1) * a->in_head_stride + a->width <= a->in_stride &&
                       v->in_row_bytes >= (int64_t)a->in_stride * 4 && a->out_off >= 0 &&
                       a->out_off + (int64_t)(a->heads - 1) * a->out_head_stride + a->width <= a->out_stride &&
                       v->out_row_bytes >= (int64_t)a->out_stride * 4,
                   "rotate_heads: rows too short for %d stretches at the offsets named", a->heads);
    PICOLM_REQUIRE(v->in != v->out || (a->in_stride == a->out_stride && a->in_off == a->out_off && a->in_head_stride == a->out_head_stride &&
                                       !a->more_heads && !a->norm_weight),
                   "rotate_heads: in place needs equal offsets and strides, and no further stretches");
    PICOLM_REQUIRE(a->more_heads >= 0 && (!a->more_heads ||
                                          (a->more_in_head_stride >= (a->more_heads > 1 ? a->width : 0) &&
                                           a->more_out_head_stride >= (a->more_heads > 1 ? a->width : 0) && a->more_in_off >= 0 &&
                                           a->more_in_off + (int64_t)(a->more_heads - 1) * a->more_in_head_stride + a->width <= a->in_stride &&
                                           a->more_out_off >= 0 &&
                                           a->more_out_off + (int64_t)(a->more_heads - 1) * a->more_out_head_stride + a->width <= a->out_stride)),
                   "rotate_heads: rows too short for %d further stretches at the offsets named", a->more_heads);
    PICOLM_REQUIRE(!a->norm_weight || (a->norm_width > 0 && a->norm_eps > 0.f && a->norm_in_off >= 0 && a->norm_in_off + a->norm_width <= a->in_stride &&
                                       a->norm_out_off >= 0 && a->norm_out_off + a->norm_width <= a->out_stride),
                   "rotate_heads: rows too short for a normed stretch of %d columns at the offsets named", a->norm_width);
    for (int i = 0; i < v->n_seq; ++i)
        PICOLM_REQUIRE(v->recording || v->pos0[i] + v->n_new[i] <= a->table_positions,
                       "rotate_heads: sequence %d reaches position %d, the tables hold %d", i, v->pos0[i] + v->n_new[i], a->table_positions);
    if (v->rows <= 0) return 0;
    rotate_heads_kernel<<<v->rows, 256, 0, v->stream>>>(*a, (const float*)v->in, (float*)v->out, v->tok_pos);
    PICOLM_LAUNCH_CHECK("rotate_heads");
    return 0;
}

// ---- a sum of rows -----------------------------------------------------------------------------------
__global__ void add_rows_kernel(float* __restrict__ x, const float* __restrict__ in, const float* __restrict__ vec, int W) {
    const size_t row = blockIdx.x;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        float y = x[row * W + c];
        if (in) y += in[row * W + c];
        if (vec) y += vec[c];
        x[row * W + c] = y;
    }
}

extern "C" int picolm_call_add_rows(void* user, const picolm_step_view* v) {
    const picolm_add_rows_args* a = (const picolm_add_rows_args*)user;
    VIEW_REQUIRE("add_rows", v);
    PICOLM_REQUIRE(a && a->width > 0 && v->out && (v->in || a->vec), "add_rows: nothing to add, or no rows to add to");
    PICOLM_REQUIRE(v->out_row_bytes >= a->width * 4 && (!v->in || v->in_row_bytes >= a->width * 4), "add_rows: rows too short for a width of %d",
                   a->width);
    if (v->rows <= 0) return 0;
    add_rows_kernel<<<v->rows, 256, 0, v->stream>>>((float*)v->out, (const float*)v->in, a->vec, a->width);
    PICOLM_LAUNCH_CHECK("add_rows");
    return 0;
}

// ---- two attention maps a head become one ------------------------------------------------------------
// one wave per (row, head)
__global__ void map_difference_kernel(const float* __restrict__ in, void* __restrict__ out, int out_dt, int heads, int dv, float lambda, float eps,
                                      float mult) {
    const size_t row = blockIdx.x;
    const int head = blockIdx.y * (blockDim.x / WAVE) + threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    if (head >= heads) return;
    const float* a1 = in + (row * heads + head) * 2 * dv;
    const float* a2 = a1 + dv;
    float ssq = 0.f;
    for (int c = lane; c < dv; c += WAVE) {
        const float o = a1[c] - lambda * a2[c];
        ssq += o * o;
    }
    ssq = wave_sum(ssq);
    const float k = mult / sqrtf(ssq / (float)dv + eps);
    for (int c = lane; c < dv; c += WAVE) store_from_f32(out, (row * heads + head) * dv + c, out_dt, (a1[c] - lambda * a2[c]) * k);
}

extern "C" int picolm_call_map_difference(void* user, const picolm_step_view* v) {
    const picolm_map_difference_args* a = (const picolm_map_difference_args*)user;
    VIEW_REQUIRE("map_difference", v);
    PICOLM_REQUIRE(a && a->heads > 0 && a->vdim > 0 && known_dtype(a->out_dtype) && v->in && v->out && v->in != v->out,
                   "map_difference: sizes or buffers are missing (input and output differ)");
    PICOLM_REQUIRE(v->in_row_bytes >= (int64_t)a->heads * 2 * a->vdim * 4 && v->out_row_bytes >= (int64_t)a->heads * a->vdim * elem_bytes(a->out_dtype),
                   "map_difference: rows too short for %d heads of %d", a->heads, a->vdim);
    if (v->rows <= 0) return 0;
    const int waves = 4;
    PICOLM_REQUIRE(ceil_div(a->heads, waves) <= 65535, "map_difference: %d heads exceed the grid", a->heads);
    map_difference_kernel<<<dim3(v->rows, ceil_div(a->heads, waves)), waves * WAVE, 0, v->stream>>>((const float*)v->in, v->out, a->out_dtype, a->heads,
                                                                                                 a->vdim, a->lambda, a->eps, a->mult);
    PICOLM_LAUNCH_CHECK("map_difference");
    return 0;
}

// ---- two norms of the same rows -------------------------------------------------------------------------
// a workgroup a row: the row is read once for the sum of squares and once more (from cache) for the outputs
template <typename T>
__global__ __launch_bounds__(256) void rms_pair_kernel(const float* __restrict__ x, T* __restrict__ a, T* __restrict__ b,
                                                       const float* __restrict__ w_a, const float* __restrict__ w_b, int W, float eps) {
    __shared__ float scratch[16];
    const size_t row = blockIdx.x;
    const float* xr = x + row * W;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) ss += xr[c] * xr[c];
    ss = block_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float y = xr[c] * inv;
        a[row * W + c] = from_f32<T>(y * w_a[c]);
        b[row * W + c] = from_f32<T>(y * w_b[c]);
    }
}

extern "C" int picolm_call_rms_pair(void* user, const picolm_step_view* v) {
    const picolm_rms_pair_args* a = (const picolm_rms_pair_args*)user;
    VIEW_REQUIRE("rms_pair", v);
    PICOLM_REQUIRE(a && a->w_a && a->w_b && a->width > 0 && known_dtype(a->out_dtype) && v->in && v->out && v->extra[0] && v->out != v->extra[0],
                   "rms_pair: weights or buffers are missing (the two outputs differ)");
    const int es = elem_bytes(a->out_dtype);
    PICOLM_REQUIRE(v->in_row_bytes >= a->width * 4 && v->out_row_bytes >= a->width * es && v->extra_row_bytes[0] >= a->width * es,
                   "rms_pair: rows too short for a width of %d", a->width);
    if (v->rows <= 0) return 0;
    if (a->out_dtype == PICOLM_F32)
        rms_pair_kernel<float><<<v->rows, 256, 0, v->stream>>>((const float*)v->in, (float*)v->out, (float*)v->extra[0], a->w_a, a->w_b, a->width, a->eps);
    else
        rms_pair_kernel<bf16_t><<<v->rows, 256, 0, v->stream>>>((const float*)v->in, (bf16_t*)v->out, (bf16_t*)v->extra[0], a->w_a, a->w_b, a->width,
                                                                a->eps);
    PICOLM_LAUNCH_CHECK("rms_pair");
    return 0;
}
