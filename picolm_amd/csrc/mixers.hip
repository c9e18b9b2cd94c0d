// Called operations of the library's own (mixers.h): the row-wise steps around mixers with state,
// a softmax attention with a bias by distance, a sink and a gate, a short convolution over time
// and a matrix state that is walked token by token.  Every function checks what it is handed on
// the host, then queues its kernels on the step's stream; what they do depends on device memory
// only, so a decode step that holds them can be recorded and replayed.
//
// All arithmetic is float; only rows that feed a product are written in the engine's dtype.
#include "mixers.h"

#include "api.h"
#include "common.h"
#include "attention.h"

#define VIEW_REQUIRE(who, v)                                                                                      \
    PICOLM_REQUIRE((v) && (v)->struct_bytes == (int32_t)sizeof(picolm_step_view), "%s: the step view is of another version", who)

static inline int elem_bytes(int dt) { return dt == PICOLM_F32 ? 4 : 2; }

__device__ __forceinline__ float silu_f(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// ---- the input of a pass over a looped stretch --------------------------------------------------
template <typename T>
__global__ void loop_input_kernel(float* __restrict__ x, const float* __restrict__ first, T* __restrict__ joined,
                                  const float* __restrict__ step, int W) {
    const size_t row = blockIdx.x;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        joined[row * 2 * W + c] = from_f32<T>(x[row * W + c]);
        joined[row * 2 * W + W + c] = from_f32<T>(first[row * W + c]);
        x[row * W + c] = step[c];
    }
}

extern "C" int picolm_call_loop_input(void* user, const picolm_step_view* v) {
    const picolm_loop_input_args* a = (const picolm_loop_input_args*)user;
    VIEW_REQUIRE("loop_input", v);
    PICOLM_REQUIRE(a && a->step && a->width > 0 && v->in && v->out && v->extra[0], "loop_input: buffers or the pass's vector are missing");
    PICOLM_REQUIRE(v->in_row_bytes >= a->width * 4 && v->out_row_bytes >= a->width * 4 &&
                       v->extra_row_bytes[0] >= 2 * a->width * elem_bytes(v->dtype),
                   "loop_input: rows too short for a width of %d", a->width);
    if (v->rows <= 0) return 0;
    if (v->dtype == PICOLM_F32)
        loop_input_kernel<float><<<v->rows, 256, 0, v->stream>>>((float*)v->out, (const float*)v->in, (float*)v->extra[0], a->step, a->width);
    else
        loop_input_kernel<bf16_t><<<v->rows, 256, 0, v->stream>>>((float*)v->out, (const float*)v->in, (bf16_t*)v->extra[0], a->step, a->width);
    PICOLM_LAUNCH_CHECK("loop_input");
    return 0;
}

// ---- attention with a norm of queries and keys, a bias by distance, a sink and a gate ------------
struct QkPrepare {
    const float* in;
    int in_stride, q_off, k_off, v_off;
    const float* q_norm;
    const float* k_norm;
    float eps;
    int unit_qk;
    const float* in_bias;
    const float* cos_t;
    const float* sin_t;
    int table_positions, rot_dims, rot_half;
    const int32_t* tok_pos;
    const int32_t* write_pages;
    int H, G, d, dv, maps;
    bool tiled;
};

// One wave per (token, part): a part is one of the `maps` queries of a query head, one of the `maps`
// keys of a KV head, or a value head.  Queries go, biased, turned and normed, to the rows the
// attention kernel reads (query m of a head as a row of d entries that is zero outside part m, so
// that its product with the cached key is its product with the key's part m); keys likewise to the
// token's place in its cache page, values (biased only) too (K[G][64][d], V^T[G][dv][64] as plain
// arrays, or with `tiled` in the order of the MFMA operands).
template <typename T>
__global__ void qk_norm_store_kernel(QkPrepare a, T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages) {
    const size_t row = blockIdx.x;
    const int unit = blockIdx.y, lane = threadIdx.x;
    const int H = a.H, G = a.G, d = a.d, dv = a.dv, maps = a.maps, dp = d / maps;
    const float* src = a.in + row * a.in_stride;
    if (unit < (H + G) * maps) {
        const bool is_q = unit < H * maps;
        const int part = is_q ? unit : unit - H * maps;          // (head, map) counted together
        const int at = (is_q ? a.q_off : a.k_off) + part * dp;
        const float* x = src + at;
        const float* b = a.in_bias ? a.in_bias + at : nullptr;
        const float* w = is_q ? a.q_norm : a.k_norm;
        const int half = a.rot_dims / 2;
        const int pos = a.cos_t ? min(a.tok_pos[row], a.table_positions - 1) : 0;
        const float* ct = a.cos_t ? a.cos_t + (size_t)pos * half : nullptr;
        const float* st = a.cos_t ? a.sin_t + (size_t)pos * half : nullptr;
        auto entry = [&](int i) { return b ? x[i] + b[i] : x[i]; };
        auto value = [&](int i) {
            if (!ct || i >= a.rot_dims) return entry(i);
            int j, first, second;
            if (a.rot_half) j = i < half ? i : i - half, first = j, second = j + half;
            else j = i >> 1, first = 2 * j, second = 2 * j + 1;
            const float u = entry(first), v = entry(second), c = ct[j], s = st[j];
            return i == first ? u * c - v * s : v * c + u * s;
        };
        float inv = 1.f;
        const bool norms = w || a.unit_qk;
        if (norms) {
            float ssq = 0.f;
            for (int i = lane; i < dp; i += WAVE) {
                const float y = value(i);
                ssq += y * y;
            }
            ssq = wave_sum(ssq);
            inv = 1.f / sqrtf(ssq / (float)dp + a.eps);
        }
        const int m = part % maps, lo = m * dp;
        if (is_q) {
            T* dst = q_out + (row * H * maps + part) * d;
            for (int i = lane; i < d; i += WAVE) {
                float y = 0.f;
                if (i >= lo && i < lo + dp) {
                    y = value(i - lo);
                    if (norms) y = w ? y * inv * w[i - lo] : y * inv;
                }
                dst[i] = from_f32<T>(y);
            }
        } else {
            const int head = part / maps;
            const int key = a.tok_pos[row] % PAGE_TOKENS;
            T* dst = k_pages + ((size_t)a.write_pages[row] * G + head) * PAGE_TOKENS * d;
            for (int i = lane; i < dp; i += WAVE) {
                float y = value(i);
                if (norms) y = w ? y * inv * w[i] : y * inv;
                dst[k_page_offset(key, lo + i, d, a.tiled)] = from_f32<T>(y);
            }
        }
    } else {
        const int head = unit - (H + G) * maps;
        const float* x = src + a.v_off + (size_t)head * dv;
        const float* b = a.in_bias ? a.in_bias + a.v_off + (size_t)head * dv : nullptr;
        const int key = a.tok_pos[row] % PAGE_TOKENS;
        T* dst = v_pages + ((size_t)a.write_pages[row] * G + head) * dv * PAGE_TOKENS;
        for (int i = lane; i < dv; i += WAVE) dst[v_page_offset(i, key, dv, a.tiled)] = from_f32<T>(b ? x[i] + b[i] : x[i]);
    }
}

extern "C" int picolm_call_sink_attention(void* user, const picolm_step_view* v) {
    const picolm_sink_attention_args* a = (const picolm_sink_attention_args*)user;
    VIEW_REQUIRE("sink_attention", v);
    PICOLM_REQUIRE(a && v->in && v->out && v->extra[0] && v->k_pages && v->v_pages && v->page_table,
                   "sink_attention: buffers or the cache entry are missing");
    const int H = a->n_heads, G = a->n_kv_heads, d = a->head_dim, dv = a->v_head_dim, dt = v->dtype, es = elem_bytes(dt);
    const int maps = a->maps > 1 ? a->maps : 1;
    PICOLM_REQUIRE(H > 0 && G > 0 && H % G == 0 && d > 0 && dv > 0, "sink_attention: %d heads over %d, sizes %d and %d", H, G, d, dv);
    PICOLM_REQUIRE(G == v->n_kv_heads && d == v->head_dim && dv == v->v_head_dim && v->window >= 0,
                   "sink_attention: the cache entry holds %d heads of %d and %d (window %d), the operation has %d of %d and %d", v->n_kv_heads,
                   v->head_dim, v->v_head_dim, v->window, G, d, dv);
    PICOLM_REQUIRE(v->in_row_bytes >= a->in_stride * 4 && a->q_off >= 0 && a->q_off + H * d <= a->in_stride && a->k_off >= 0 &&
                       a->k_off + G * d <= a->in_stride && a->v_off >= 0 && a->v_off + G * dv <= a->in_stride &&
                       (a->gate_off < 0 || a->gate_off + H * dv <= a->in_stride),
                   "sink_attention: the input rows of %d floats do not hold what the offsets name", a->in_stride);
    PICOLM_REQUIRE(d % maps == 0 && (maps == 1 || (a->gate_off < 0 && !a->bias)),
                   "sink_attention: %d queries a head of %d entries (with several there is no gate and no bias by distance)", maps, d);
    PICOLM_REQUIRE(v->out_row_bytes >= (int64_t)H * maps * dv * (a->out_float ? 4 : es) && v->extra_row_bytes[0] >= (int64_t)H * maps * d * es,
                   "sink_attention: output or scratch rows too short");
    PICOLM_REQUIRE(!v->kv_writes || v->write_pages, "sink_attention: no pages to write to");
    PICOLM_REQUIRE(a->window >= 0 && (v->window <= 0 || a->window <= v->window), "sink_attention: a window of %d keys over a cache entry laid out for %d",
                   a->window, v->window);
    PICOLM_REQUIRE(a->chunk >= 0, "sink_attention: stretches of %d keys", a->chunk);
    PICOLM_REQUIRE(!a->cos_table || (a->sin_table && a->table_positions > 0 && a->rot_dims > 0 && a->rot_dims % 2 == 0 && a->rot_dims <= d / maps),
                   "sink_attention: a rotation of %d entries of %d, tables for %d positions", a->rot_dims, d / maps, a->table_positions);
    PICOLM_REQUIRE((H + G) * maps + G <= 65535, "sink_attention: %d heads exceed the grid", (H + G) * maps + G);
    if (v->n_tokens <= 0) return 0;
    const float* in = (const float*)v->in;
    dim3 grid(v->n_tokens, v->kv_writes ? (H + G) * maps + G : H * maps);
    const bool mfma = dt == PICOLM_BF16 && picolm_attn_plain_mfma_takes(d, dv);      // then the pages are in the matrix-core kernel's order
    QkPrepare p = {in, a->in_stride, a->q_off, a->k_off, a->v_off, a->q_norm, a->k_norm, a->eps, a->unit_qk, a->in_bias, a->cos_table,
                   a->sin_table, a->table_positions, a->rot_dims, a->rot_half, v->tok_pos, v->write_pages, H, G, d, dv, maps, mfma};
    if (dt == PICOLM_F32)
        qk_norm_store_kernel<float><<<grid, WAVE, 0, v->stream>>>(p, (float*)v->extra[0], (float*)v->k_pages, (float*)v->v_pages);
    else
        qk_norm_store_kernel<bf16_t><<<grid, WAVE, 0, v->stream>>>(p, (bf16_t*)v->extra[0], (bf16_t*)v->k_pages, (bf16_t*)v->v_pages);
    PICOLM_LAUNCH_CHECK("sink_attention (norm and cache write)");
    picolm_attn_extras x;
    x.v_head_dim = dv;
    x.bias = a->bias;
    x.bias_rows = a->bias_rows;
    x.sink = a->sink;
    x.gate = a->gate_off >= 0 ? in + a->gate_off : nullptr;
    x.gate_stride = a->in_stride;
    x.mask_window = a->window;
    x.mask_chunk = a->chunk;
    x.out_float = a->out_float;
    const int HM = H * maps;
    if (mfma && v->is_decode)
        return picolm_attn_decode_plain_mfma(v->extra[0], v->k_pages, v->v_pages, v->out, v->partial, v->n_seq, v->chunk_list, v->n_chunks,
                                             v->pages_per_chunk, v->most_chunks, v->seq_pos0, v->page_table, v->max_pages, v->ring_pages, HM,
                                             G, d, v->window, a->scale, &x, v->stream);
    if (mfma) {
        PICOLM_REQUIRE(v->tile_seq && v->tile_rows == picolm_attn_plain_mfma_tile_rows(), "sink_attention: the step has no tiles of %d rows",
                       picolm_attn_plain_mfma_tile_rows());
        return picolm_attn_prefill_plain_mfma(v->extra[0], v->k_pages, v->v_pages, v->out, v->tile_seq, v->tile_q0, v->n_tiles, v->seq_slot,
                                              v->seq_pos0, v->seq_nnew, v->cu_seqlens, v->page_table, v->max_pages, v->ring_pages, HM, G, d,
                                              v->window, a->scale, &x, v->stream);
    }
    if (v->is_decode)
        return picolm_attn_decode_plain(v->extra[0], v->k_pages, v->v_pages, v->out, v->partial, dt, v->n_seq, v->chunk_list, v->n_chunks,
                                        v->pages_per_chunk, v->most_chunks, v->seq_pos0, v->page_table, v->max_pages, v->ring_pages, HM, G, d,
                                        v->window, a->scale, &x, v->stream);
    PICOLM_REQUIRE(v->tile_seq && v->tile_rows == picolm_attn_prefill_tile_rows(), "sink_attention: the step has no tiles of %d rows",
                   picolm_attn_prefill_tile_rows());
    return picolm_attn_prefill_plain(v->extra[0], v->k_pages, v->v_pages, v->out, dt, v->tile_seq, v->tile_q0, v->n_tiles, v->seq_slot,
                                     v->seq_pos0, v->seq_nnew, v->cu_seqlens, v->page_table, v->max_pages, v->ring_pages, HM, G, d, v->window,
                                     a->scale, &x, v->stream);
}

// ---- a short causal convolution over time ---------------------------------------------------------
#define CONV_MAX_TAPS 16

// thread = (row, channel): the inputs of the taps come from the step's rows where the sequence has
// them there, from the slot's state (the last taps - 1 inputs before the step, oldest first) else
__global__ void short_conv_kernel(const float* __restrict__ in, int in_stride, int in_off, float* __restrict__ out, int out_stride,
                                  int out_off, const float* __restrict__ state, int64_t slot_floats, const float* __restrict__ weight,
                                  const float* __restrict__ bias, int C, int taps, int act, const int32_t* __restrict__ tok_seq,
                                  const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_slot) {
    const int row = blockIdx.x;
    const int seq = tok_seq[row], l = row - cu_seqlens[seq];
    const float* st = state + (size_t)seq_slot[seq] * slot_floats;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
        float acc = bias ? bias[c] : 0.f;
        for (int j = taps - 1; j >= 0; --j) {       // oldest first
            const float xv = j <= l ? in[(size_t)(row - j) * in_stride + in_off + c] : st[(size_t)(taps - 1 + l - j) * C + c];
            acc += weight[(size_t)c * taps + taps - 1 - j] * xv;
        }
        out[(size_t)row * out_stride + out_off + c] = act == 1 ? silu_f(acc) : acc;
    }
}

// thread = (sequence, channel): the state after the step, read whole before any of it is written
__global__ void short_conv_state_kernel(const float* __restrict__ in, int in_stride, int in_off, float* __restrict__ state,
                                        int64_t slot_floats, int C, int taps, const int32_t* __restrict__ cu_seqlens,
                                        const int32_t* __restrict__ seq_slot) {
    const int seq = blockIdx.x;
    const int row0 = cu_seqlens[seq], n = cu_seqlens[seq + 1] - row0;
    float* st = state + (size_t)seq_slot[seq] * slot_floats;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
        float keep[CONV_MAX_TAPS - 1];
#pragma unroll
        for (int i = 0; i < CONV_MAX_TAPS - 1; ++i) {
            if (i >= taps - 1) break;
            const int p = n - (taps - 1) + i;       // place among the step's tokens; negative: older than the step
            keep[i] = p >= 0 ? in[(size_t)(row0 + p) * in_stride + in_off + c] : st[(size_t)(i + n) * C + c];
        }
#pragma unroll
        for (int i = 0; i < CONV_MAX_TAPS - 1; ++i) {
            if (i >= taps - 1) break;
            st[(size_t)i * C + c] = keep[i];
        }
    }
}

extern "C" int picolm_call_short_conv(void* user, const picolm_step_view* v) {
    const picolm_short_conv_args* a = (const picolm_short_conv_args*)user;
    VIEW_REQUIRE("short_conv", v);
    PICOLM_REQUIRE(a && a->weight && v->in && v->out && v->in != v->out, "short_conv: weights or buffers are missing (input and output differ)");
    PICOLM_REQUIRE(a->channels > 0 && a->taps >= 1 && a->taps <= CONV_MAX_TAPS, "short_conv: %d channels, %d taps (up to %d)", a->channels,
                   a->taps, CONV_MAX_TAPS);
    PICOLM_REQUIRE(a->in_off >= 0 && a->in_off + a->channels <= a->in_stride && v->in_row_bytes >= a->in_stride * 4 && a->out_off >= 0 &&
                       a->out_off + a->channels <= a->out_stride && v->out_row_bytes >= a->out_stride * 4,
                   "short_conv: rows too short for %d channels at the offsets named", a->channels);
    const int64_t need = (a->state_off + (int64_t)(a->taps - 1) * a->channels) * 4;
    PICOLM_REQUIRE(a->taps == 1 || (v->state && a->state_off >= 0 && need <= v->state_bytes_per_slot),
                   "short_conv: the state of a slot has %lld bytes, the last inputs need %lld", (long long)v->state_bytes_per_slot, (long long)need);
    if (v->n_tokens <= 0) return 0;
    const int64_t slot_floats = v->state_bytes_per_slot / 4;
    float* state = v->state ? (float*)v->state + a->state_off : nullptr;
    const int by = std::min(ceil_div(a->channels, 256), 1024);
    short_conv_kernel<<<dim3(v->n_tokens, by), 256, 0, v->stream>>>((const float*)v->in, a->in_stride, a->in_off, (float*)v->out, a->out_stride,
                                                                    a->out_off, state, slot_floats, a->weight, a->bias, a->channels, a->taps,
                                                                    a->act, v->tok_seq, v->cu_seqlens, v->seq_slot);
    PICOLM_LAUNCH_CHECK("short_conv");
    if (a->taps > 1) {
        short_conv_state_kernel<<<dim3(v->n_seq, by), 256, 0, v->stream>>>((const float*)v->in, a->in_stride, a->in_off, state, slot_floats,
                                                                           a->channels, a->taps, v->cu_seqlens, v->seq_slot);
        PICOLM_LAUNCH_CHECK("short_conv (state)");
    }
    return 0;
}

// ---- a matrix state per head, walked token by token -------------------------------------------------
// Before the walk, per token: q and k made unit vectors (and q scaled), in place, and every head's
// decay and strength from their pre-activations.
__global__ void state_scan_prepare_kernel(const float* __restrict__ in, int in_stride, int a_off, int w_off, float* __restrict__ qkv,
                                          int qkv_stride, int q_off, int k_off, float* __restrict__ aw, const float* __restrict__ A_log,
                                          const float* __restrict__ dt_bias, int rule, int heads, int key_heads, int key_dim, int unit_qk,
                                          float unit_eps, float q_scale) {
    const size_t row = blockIdx.x;
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, n_waves = blockDim.x / WAVE;
    if (unit_qk || q_scale != 1.f)
        for (int u = wave; u < 2 * key_heads; u += n_waves) {
            const bool is_q = u < key_heads;
            if (!is_q && !unit_qk) continue;
            float* x = qkv + row * qkv_stride + (is_q ? q_off + (size_t)u * key_dim : k_off + (size_t)(u - key_heads) * key_dim);
            float mult = is_q ? q_scale : 1.f;
            if (unit_qk) {
                float ssq = 0.f;
                for (int i = lane; i < key_dim; i += WAVE) ssq += x[i] * x[i];
                ssq = wave_sum(ssq);
                mult *= 1.f / sqrtf(ssq + unit_eps);
            }
            for (int i = lane; i < key_dim; i += WAVE) x[i] *= mult;
        }
    for (int h = threadIdx.x; h < heads; h += blockDim.x) {
        const float ra = in[row * in_stride + a_off + h], rw = in[row * in_stride + w_off + h];
        const float bias = dt_bias ? dt_bias[h] : 0.f;
        aw[row * 2 * heads + h] = expf(-expf(A_log[h]) * softplus_f(ra + bias));
        aw[row * 2 * heads + heads + h] = rule == 0 ? softplus_f(rw + bias) : sigmoid_f(rw);
    }
}

#define SCAN_TB 16       // tokens whose q, k, v wait in LDS at a time

struct ScanArgs {
    const float* qkv;
    const float* aw;
    float* out;
    float* state;
    const float* skip;
    const int32_t* cu_seqlens;
    const int32_t* seq_slot;
    int64_t slot_floats;
    int qkv_stride, q_off, k_off, v_off;
    int rule, heads, key_heads, key_dim, value_dim;
    int R, kpt, n_waves, n_cb;
    // mode 0: whole sequences, from and to the slot's state.  A long prompt is walked in chunks of
    // chunk_len tokens side by side instead: mode 1 leaves every chunk's effect on a state as
    // (N, M) with  S_end = M S_start + N  (the update is affine in S: the chunk is walked once from
    // S = 0 with its values, which gives N, and with the delta rule once more from S = I without
    // values, which gives M as key_dim more columns; the outer-product rule's M is the product of
    // the chunk's decays); scan_carry_kernel then takes the states from chunk to chunk; mode 3
    // walks every chunk from its start state and writes the outputs.
    int mode, chunk_len, chunks_per_seq, ws_cols;
    float* ws;          // [sequence][chunk][head][key_dim][ws_cols]: N | M | S_start
};

__device__ __forceinline__ float* scan_ws(const ScanArgs& a, int seq, int chunk, int head) {
    return a.ws + (((size_t)seq * a.chunks_per_seq + chunk) * a.heads + head) * a.key_dim * a.ws_cols;
}

// One workgroup per (sequence, head, block of value columns).  A column of the state lies in the
// registers of R lanes, up to SCAN_KPT rows each (row i R + r with lane r), so that both sums over
// the rows of a column, the read-back along k and the read-out along q, are short chains in a lane
// and a few steps across lanes.  (A whole column of 128 rows in one lane was measured too: the
// chains of 128 dependent multiply-adds and the fewer waves made the walk 2.4 times slower.)
// Lane = r * CW + column within the wave (CW = 64 / R columns a wave).
#define SCAN_KPT 16      // rows of the state a thread keeps in registers
template <int R>
__global__ __launch_bounds__(256) void state_scan_kernel(ScanArgs a) {
    extern __shared__ float scan_lds[];
    constexpr int CW = WAVE / R;
    const int kpt = a.kpt, kd = kpt * R, CB = a.n_waves * CW;
    float* ks = scan_lds;                    // [TB][kd]
    float* qs = ks + SCAN_TB * kd;           // [TB][kd]
    float* vs = qs + SCAN_TB * kd;           // [TB][CB]
    float* aws = vs + SCAN_TB * CB;          // [TB][2]
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int cb = blockIdx.x % a.n_cb, head = (blockIdx.x / a.n_cb) % a.heads, unit = blockIdx.x / (a.n_cb * a.heads);
    const int seq = a.mode ? unit / a.chunks_per_seq : unit, chunk = a.mode ? unit % a.chunks_per_seq : 0;
    int row0 = a.cu_seqlens[seq], row1 = a.cu_seqlens[seq + 1];
    if (a.mode) {
        row0 += chunk * a.chunk_len;
        if (row0 >= row1) return;               // (the whole workgroup: the sequence has fewer chunks)
        row1 = min(row1, row0 + a.chunk_len);
    }
    const int r = lane / CW, col = wave * CW + lane % CW, j = cb * CB + col;
    const int n_cols = a.mode == 1 ? a.ws_cols - a.value_dim : a.value_dim;      // mode 1: the columns of N and of M
    const bool valid = j < n_cols;
    const int kh = head / (a.heads / a.key_heads);
    float* st = a.state + (size_t)a.seq_slot[seq] * a.slot_floats + (size_t)head * a.key_dim * a.value_dim;
    float* ws = a.mode ? scan_ws(a, seq, chunk, head) : nullptr;
    float S[SCAN_KPT];
#pragma unroll
    for (int i = 0; i < SCAN_KPT; ++i) {
        const int kr = i * R + r;
        const bool in = i < kpt && valid && kr < a.key_dim;
        if (a.mode == 0) S[i] = in ? st[(size_t)kr * a.value_dim + j] : 0.f;
        else if (a.mode == 1) S[i] = in && j - a.value_dim == kr ? 1.f : 0.f;
        else S[i] = in ? ws[(size_t)kr * a.ws_cols + (a.ws_cols - a.value_dim) + j] : 0.f;
    }
    const float skip = a.skip ? a.skip[head] : 0.f;
    for (int b0 = row0; b0 < row1; b0 += SCAN_TB) {
        const int nb = min(SCAN_TB, row1 - b0);
        __syncthreads();
        for (int idx = tid; idx < nb * kd; idx += blockDim.x) {
            const int t = idx / kd, i = idx % kd;
            const float* src = a.qkv + (size_t)(b0 + t) * a.qkv_stride + (size_t)kh * a.key_dim + i;
            ks[idx] = i < a.key_dim ? src[a.k_off] : 0.f;
            qs[idx] = i < a.key_dim ? src[a.q_off] : 0.f;
        }
        for (int idx = tid; idx < nb * CB; idx += blockDim.x) {
            const int t = idx / CB, c = cb * CB + idx % CB;
            vs[idx] = c < a.value_dim ? a.qkv[(size_t)(b0 + t) * a.qkv_stride + a.v_off + (size_t)head * a.value_dim + c] : 0.f;
        }
        for (int idx = tid; idx < nb * 2; idx += blockDim.x)
            aws[idx] = a.aw[(size_t)(b0 + idx / 2) * 2 * a.heads + (idx % 2) * a.heads + head];
        __syncthreads();
        for (int t = 0; t < nb; ++t) {
            const float av = aws[2 * t], wv = aws[2 * t + 1], vv = vs[t * CB + col];
            const float* k = ks + t * kd + r;
            const float* q = qs + t * kd + r;
            float o = 0.f;
            if (a.rule == 1) {
                float dot = 0.f;
#pragma unroll
                for (int i = 0; i < SCAN_KPT; ++i)
                    if (i < kpt) {
                        S[i] *= av;
                        dot += S[i] * k[i * R];
                    }
                for (int off = CW; off < WAVE; off <<= 1) dot += __shfl_xor(dot, off, WAVE);
                const float u = wv * (vv - dot);
#pragma unroll
                for (int i = 0; i < SCAN_KPT; ++i)
                    if (i < kpt) {
                        S[i] += k[i * R] * u;
                        o += S[i] * q[i * R];
                    }
            } else {
                const float wvv = wv * vv;
#pragma unroll
                for (int i = 0; i < SCAN_KPT; ++i)
                    if (i < kpt) {
                        S[i] = av * S[i] + k[i * R] * wvv;
                        o += S[i] * q[i * R];
                    }
            }
            for (int off = CW; off < WAVE; off <<= 1) o += __shfl_xor(o, off, WAVE);
            if (r == 0 && valid && a.mode != 1)
                a.out[(size_t)(b0 + t) * a.heads * a.value_dim + (size_t)head * a.value_dim + j] = o + skip * vv;
        }
    }
    if (a.mode == 3) return;
#pragma unroll
    for (int i = 0; i < SCAN_KPT; ++i) {
        const int kr = i * R + r;
        if (i < kpt && valid && kr < a.key_dim) {
            if (a.mode == 0) st[(size_t)kr * a.value_dim + j] = S[i];
            else ws[(size_t)kr * a.ws_cols + j] = S[i];
        }
    }
}

// From chunk to chunk: S_start of every chunk, and the state after the last one to the slot.  One
// workgroup per (sequence, head, CARRY_COLS value columns); the columns of S lie in LDS.  Few
// columns a workgroup, so that many workgroups share the one walk that is left in order.  The
// outer-product rule's decays of all chunks are multiplied up first, a wave a chunk.  (The delta
// rule's M passed through LDS in tiles of 32 columns was measured too: three times slower than rows
// of M read from global memory by the threads that share them.)
#define CARRY_COLS 4
#define CARRY_MAX (PICOLM_STATE_SCAN_MAX_KEY_DIM * CARRY_COLS / 256)      // elements a thread holds
__global__ __launch_bounds__(256) void scan_carry_kernel(ScanArgs a) {
    extern __shared__ float carry_lds[];      // S [key_dim][CARRY_COLS] | decays [chunks_per_seq]
    float* decays = carry_lds + a.key_dim * CARRY_COLS;
    const int n_cb = (a.value_dim + CARRY_COLS - 1) / CARRY_COLS;
    const int cb = blockIdx.x % n_cb, head = (blockIdx.x / n_cb) % a.heads, seq = blockIdx.x / (n_cb * a.heads);
    const int row0 = a.cu_seqlens[seq], row1 = a.cu_seqlens[seq + 1];
    const int n_chunks = (row1 - row0 + a.chunk_len - 1) / a.chunk_len;
    const int n_elem = a.key_dim * CARRY_COLS, s_off = a.ws_cols - a.value_dim;
    float* st = a.state + (size_t)a.seq_slot[seq] * a.slot_floats + (size_t)head * a.key_dim * a.value_dim;
    float next[CARRY_MAX];
    for (int e = threadIdx.x; e < n_elem; e += 256) {
        const int i = e / CARRY_COLS, j = cb * CARRY_COLS + e % CARRY_COLS;
        carry_lds[e] = j < a.value_dim ? st[(size_t)i * a.value_dim + j] : 0.f;
    }
    if (a.rule == 0) {
        const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
        for (int c = wave; c < n_chunks; c += 256 / WAVE) {
            const int t0 = row0 + c * a.chunk_len, t1 = min(row1, t0 + a.chunk_len);
            float p = 1.f;
            for (int t = t0 + lane; t < t1; t += WAVE) p *= a.aw[(size_t)t * 2 * a.heads + head];
            for (int off = 1; off < WAVE; off <<= 1) p *= __shfl_xor(p, off, WAVE);
            if (lane == 0) decays[c] = p;
        }
    }
    __syncthreads();
    for (int c = 0; c < n_chunks; ++c) {
        float* ws = scan_ws(a, seq, c, head);
        // S_start of the chunk, and N as the start of the sums
#pragma unroll
        for (int n = 0; n < CARRY_MAX; ++n) {
            const int e = threadIdx.x + n * 256;
            if (e >= n_elem) break;
            const int i = e / CARRY_COLS, j = cb * CARRY_COLS + e % CARRY_COLS;
            const float s = carry_lds[e];
            if (j < a.value_dim) ws[(size_t)i * a.ws_cols + s_off + j] = s;
            next[n] = j < a.value_dim ? ws[(size_t)i * a.ws_cols + j] : 0.f;
            if (a.rule == 0) next[n] += decays[c] * s;
        }
        if (a.rule == 1) {
#pragma unroll
            for (int n = 0; n < CARRY_MAX; ++n) {
                const int e = threadIdx.x + n * 256;
                if (e >= n_elem) break;
                const int i = e / CARRY_COLS, jj = e % CARRY_COLS;
                const float* m = ws + (size_t)i * a.ws_cols + a.value_dim;      // row i of M: the threads of a row read it together
                float acc0 = 0.f, acc1 = 0.f;
                int k = 0;
                for (; k + 1 < a.key_dim; k += 2) {
                    acc0 += m[k] * carry_lds[k * CARRY_COLS + jj];
                    acc1 += m[k + 1] * carry_lds[(k + 1) * CARRY_COLS + jj];
                }
                if (k < a.key_dim) acc0 += m[k] * carry_lds[k * CARRY_COLS + jj];
                next[n] += acc0 + acc1;
            }
        }
        __syncthreads();
#pragma unroll
        for (int n = 0; n < CARRY_MAX; ++n) {
            const int e = threadIdx.x + n * 256;
            if (e < n_elem) carry_lds[e] = next[n];
        }
        __syncthreads();
    }
    for (int e = threadIdx.x; e < n_elem; e += 256) {
        const int i = e / CARRY_COLS, j = cb * CARRY_COLS + e % CARRY_COLS;
        if (j < a.value_dim) st[(size_t)i * a.value_dim + j] = carry_lds[e];
    }
}

// scratch of the chunked walk: one allocation of the process that grows to the largest request
// (prefill steps are not recorded, so it never changes under a recorded step)
static float* g_scan_ws = nullptr;
static size_t g_scan_ws_floats = 0;
static int scan_workspace(size_t floats, float** out) {
    if (floats > g_scan_ws_floats) {
        hipError_t e = g_scan_ws ? hipFree(g_scan_ws) : hipSuccess;
        g_scan_ws = nullptr, g_scan_ws_floats = 0;
        if (e == hipSuccess) e = hipMalloc((void**)&g_scan_ws, floats * sizeof(float));
        PICOLM_REQUIRE(e == hipSuccess, "state_scan: %zu bytes of scratch for the chunked walk: %s", floats * sizeof(float), hipGetErrorString(e));
        g_scan_ws_floats = floats;
    }
    *out = g_scan_ws;
    return 0;
}
#define SCAN_CHUNK_TOKENS 64            // a chunk of the chunked walk, doubled while the scratch would pass the limit
#define SCAN_CHUNKED_FROM 256           // new tokens of a sequence from which a step is walked in chunks
#define SCAN_WS_LIMIT_FLOATS ((size_t)1 << 30)

extern "C" int picolm_call_state_scan(void* user, const picolm_step_view* v) {
    const picolm_state_scan_args* a = (const picolm_state_scan_args*)user;
    VIEW_REQUIRE("state_scan", v);
    PICOLM_REQUIRE(a && a->A_log && v->in && v->out && v->extra[0] && v->extra[1] && v->state, "state_scan: buffers, state or constants are missing");
    const int heads = a->n_heads, kh = a->n_key_heads, kd = a->key_dim, vd = a->value_dim;
    PICOLM_REQUIRE((a->rule == 0 || a->rule == 1) && heads > 0 && kh > 0 && heads % kh == 0 && kd > 0 && kd <= PICOLM_STATE_SCAN_MAX_KEY_DIM && vd > 0,
                   "state_scan: rule %d, %d heads over %d, keys of %d (up to %d), values of %d", a->rule, heads, kh, kd,
                   PICOLM_STATE_SCAN_MAX_KEY_DIM, vd);
    PICOLM_REQUIRE(a->a_off >= 0 && a->a_off + heads <= a->in_stride && a->w_off >= 0 && a->w_off + heads <= a->in_stride &&
                       v->in_row_bytes >= a->in_stride * 4,
                   "state_scan: the input rows of %d floats do not hold a decay and a strength per head", a->in_stride);
    PICOLM_REQUIRE(a->q_off >= 0 && a->q_off + kh * kd <= a->qkv_stride && a->k_off >= 0 && a->k_off + kh * kd <= a->qkv_stride && a->v_off >= 0 &&
                       a->v_off + heads * vd <= a->qkv_stride && v->extra_row_bytes[0] >= a->qkv_stride * 4,
                   "state_scan: the rows of %d floats do not hold q, k and v at the offsets named", a->qkv_stride);
    PICOLM_REQUIRE(v->extra_row_bytes[1] >= 2 * heads * 4 && v->out_row_bytes >= heads * vd * 4, "state_scan: scratch or output rows too short");
    const int64_t need = (a->state_off + (int64_t)heads * kd * vd) * 4;
    PICOLM_REQUIRE(a->state_off >= 0 && need <= v->state_bytes_per_slot, "state_scan: the state of a slot has %lld bytes, the matrices need %lld",
                   (long long)v->state_bytes_per_slot, (long long)need);
    if (v->n_tokens <= 0) return 0;
    state_scan_prepare_kernel<<<v->n_tokens, 256, 0, v->stream>>>((const float*)v->in, a->in_stride, a->a_off, a->w_off, (float*)v->extra[0],
                                                                  a->qkv_stride, a->q_off, a->k_off, (float*)v->extra[1], a->A_log, a->dt_bias,
                                                                  a->rule, heads, kh, kd, a->unit_qk, a->unit_eps,
                                                                  a->q_scale != 0.f ? a->q_scale : 1.f);
    PICOLM_LAUNCH_CHECK("state_scan (prepare)");
    ScanArgs s;
    s.qkv = (const float*)v->extra[0];
    s.aw = (const float*)v->extra[1];
    s.out = (float*)v->out;
    s.state = (float*)v->state + a->state_off;
    s.skip = a->skip;
    s.cu_seqlens = v->cu_seqlens;
    s.seq_slot = v->seq_slot;
    s.slot_floats = v->state_bytes_per_slot / 4;
    s.qkv_stride = a->qkv_stride;
    s.q_off = a->q_off;
    s.k_off = a->k_off;
    s.v_off = a->v_off;
    s.rule = a->rule;
    s.heads = heads;
    s.key_heads = kh;
    s.key_dim = kd;
    s.value_dim = vd;
    int R = 1;
    while (R * SCAN_KPT < kd) R *= 2;           // (up to 16 for keys of PICOLM_STATE_SCAN_MAX_KEY_DIM = 256)
    s.R = R;
    s.kpt = ceil_div(kd, R);
    s.mode = 0, s.chunk_len = 0, s.chunks_per_seq = 1, s.ws_cols = 0, s.ws = nullptr;
    const int CW = WAVE / R;
    auto launch = [&](int units, int n_cols) -> int {
        // few units: one wave a workgroup, so that more workgroups share the walk; many: up to four
        int n_waves = std::min(4, ceil_div(n_cols, CW));
        if ((int64_t)units * heads * ceil_div(n_cols, n_waves * CW) < 1024) n_waves = 1;
        s.n_waves = n_waves;
        s.n_cb = ceil_div(n_cols, n_waves * CW);
        const int64_t blocks = (int64_t)units * heads * s.n_cb;
        PICOLM_REQUIRE(blocks < (1ll << 31), "state_scan: %lld workgroups exceed the grid", (long long)blocks);
        const size_t lds = sizeof(float) * SCAN_TB * ((size_t)2 * s.kpt * R + n_waves * CW + 2);
        const dim3 grid((unsigned)blocks), block(n_waves * WAVE);
        if (R == 1) state_scan_kernel<1><<<grid, block, lds, v->stream>>>(s);
        else if (R == 2) state_scan_kernel<2><<<grid, block, lds, v->stream>>>(s);
        else if (R == 4) state_scan_kernel<4><<<grid, block, lds, v->stream>>>(s);
        else if (R == 8) state_scan_kernel<8><<<grid, block, lds, v->stream>>>(s);
        else state_scan_kernel<16><<<grid, block, lds, v->stream>>>(s);
        PICOLM_LAUNCH_CHECK("state_scan");
        return 0;
    };
    int most_new = 0;
    if (!v->is_decode && !v->recording && v->n_new)
        for (int i = 0; i < v->n_seq; ++i) most_new = std::max(most_new, v->n_new[i]);
    if (most_new < SCAN_CHUNKED_FROM) return launch(v->n_seq, vd);
    // the chunked walk of a long prompt
    s.ws_cols = 2 * vd + (a->rule == 1 ? kd : 0);
    s.chunk_len = SCAN_CHUNK_TOKENS;
    auto ws_floats = [&]() { return (size_t)v->n_seq * ceil_div(most_new, s.chunk_len) * heads * kd * s.ws_cols; };
    while ((ws_floats() > SCAN_WS_LIMIT_FLOATS || ceil_div(most_new, s.chunk_len) > 2048) && s.chunk_len < most_new) s.chunk_len *= 2;
    s.chunks_per_seq = ceil_div(most_new, s.chunk_len);
    if (s.chunks_per_seq < 2) return launch(v->n_seq, vd);
    if (scan_workspace(ws_floats(), &s.ws)) return -1;
    PICOLM_REQUIRE((int64_t)v->n_seq * s.chunks_per_seq < (1 << 24), "state_scan: %d sequences of %d chunks", v->n_seq, s.chunks_per_seq);
    s.mode = 1;
    if (launch(v->n_seq * s.chunks_per_seq, s.ws_cols - vd)) return -1;
    const int64_t carry_blocks = (int64_t)v->n_seq * heads * ceil_div(vd, CARRY_COLS);
    PICOLM_REQUIRE(carry_blocks < (1ll << 31), "state_scan: %lld workgroups exceed the grid", (long long)carry_blocks);
    const size_t carry_lds = sizeof(float) * ((size_t)kd * CARRY_COLS + s.chunks_per_seq);
    PICOLM_REQUIRE(carry_lds <= 64 * 1024, "state_scan: %d chunks a sequence need %zu bytes of LDS", s.chunks_per_seq, carry_lds);
    scan_carry_kernel<<<(unsigned)carry_blocks, 256, carry_lds, v->stream>>>(s);
    PICOLM_LAUNCH_CHECK("state_scan (carry)");
    s.mode = 3;
    return launch(v->n_seq * s.chunks_per_seq, vd);
}

// ---- RMS norm in equal parts of a row, with a gate ---------------------------------------------------
// one wave per (row, part)
template <typename T>
__global__ void gated_norm_kernel(const float* __restrict__ x, const float* __restrict__ gate, int gate_stride, int gate_off,
                                  T* __restrict__ out, const float* __restrict__ weight, int weight_len, int width, int group, float eps,
                                  int gate_first, int64_t n_units) {
    const int64_t unit = (int64_t)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    const int lane = threadIdx.x % WAVE;
    if (unit >= n_units) return;
    const int n_groups = width / group;
    const size_t row = unit / n_groups;
    const int c0 = (int)(unit % n_groups) * group;
    const float* xr = x + row * width + c0;
    const float* gr = gate ? gate + row * gate_stride + gate_off + c0 : nullptr;
    float ssq = 0.f;
    for (int c = lane; c < group; c += WAVE) {
        float xv = xr[c];
        if (gr && gate_first) xv *= silu_f(gr[c]);
        ssq += xv * xv;
    }
    ssq = wave_sum(ssq);
    const float inv = 1.f / sqrtf(ssq / (float)group + eps);
    for (int c = lane; c < group; c += WAVE) {
        float xv = xr[c];
        if (gr && gate_first) xv *= silu_f(gr[c]);
        float y = xv * inv * weight[(c0 + c) % weight_len];
        if (gr && !gate_first) y *= silu_f(gr[c]);
        out[row * width + c0 + c] = from_f32<T>(y);
    }
}

// the same with a workgroup per (row, part), for parts of a thousand columns and more
template <typename T>
__global__ __launch_bounds__(1024) void gated_norm_wide_kernel(const float* __restrict__ x, const float* __restrict__ gate, int gate_stride,
                                                              int gate_off, T* __restrict__ out, const float* __restrict__ weight,
                                                              int weight_len, int width, int group, float eps, int gate_first) {
    __shared__ float scratch[16];
    const int n_groups = width / group;
    const size_t row = blockIdx.x / n_groups;
    const int c0 = (int)(blockIdx.x % n_groups) * group;
    const float* xr = x + row * width + c0;
    const float* gr = gate ? gate + row * gate_stride + gate_off + c0 : nullptr;
    float ssq = 0.f;
    for (int c = threadIdx.x; c < group; c += blockDim.x) {
        float xv = xr[c];
        if (gr && gate_first) xv *= silu_f(gr[c]);
        ssq += xv * xv;
    }
    ssq = block_sum(ssq, scratch);
    const float inv = 1.f / sqrtf(ssq / (float)group + eps);
    for (int c = threadIdx.x; c < group; c += blockDim.x) {
        float xv = xr[c];
        if (gr && gate_first) xv *= silu_f(gr[c]);
        float y = xv * inv * weight[(c0 + c) % weight_len];
        if (gr && !gate_first) y *= silu_f(gr[c]);
        out[row * width + c0 + c] = from_f32<T>(y);
    }
}

extern "C" int picolm_call_gated_norm(void* user, const picolm_step_view* v) {
    const picolm_gated_norm_args* a = (const picolm_gated_norm_args*)user;
    VIEW_REQUIRE("gated_norm", v);
    PICOLM_REQUIRE(a && a->weight && v->in && v->out, "gated_norm: weights or buffers are missing");
    PICOLM_REQUIRE(a->width > 0 && a->group > 0 && a->width % a->group == 0 && a->weight_len > 0, "gated_norm: a width of %d in parts of %d",
                   a->width, a->group);
    PICOLM_REQUIRE(v->in_row_bytes >= a->width * 4 && v->out_row_bytes >= a->width * elem_bytes(v->dtype), "gated_norm: rows too short");
    PICOLM_REQUIRE(!v->extra[0] || (a->gate_off >= 0 && a->gate_off + a->width <= a->gate_stride && v->extra_row_bytes[0] >= a->gate_stride * 4),
                   "gated_norm: the gate's rows of %d floats do not hold %d at %d", a->gate_stride, a->width, a->gate_off);
    if (v->rows <= 0) return 0;
    const int64_t n_units = (int64_t)v->rows * (a->width / a->group);
    PICOLM_REQUIRE(n_units < (1ll << 31), "gated_norm: %lld workgroups exceed the grid", (long long)n_units);
    if (a->group >= 1024) {
        // few rows (a decode step): more threads a part, so that a thread's loads, each of which it waits for, are few
        const int threads = n_units < 1024 ? 1024 : 256;
        if (v->dtype == PICOLM_F32)
            gated_norm_wide_kernel<float><<<(unsigned)n_units, threads, 0, v->stream>>>((const float*)v->in, (const float*)v->extra[0], a->gate_stride,
                                                                                    a->gate_off, (float*)v->out, a->weight, a->weight_len,
                                                                                    a->width, a->group, a->eps, a->gate_first);
        else
            gated_norm_wide_kernel<bf16_t><<<(unsigned)n_units, threads, 0, v->stream>>>((const float*)v->in, (const float*)v->extra[0],
                                                                                     a->gate_stride, a->gate_off, (bf16_t*)v->out, a->weight,
                                                                                     a->weight_len, a->width, a->group, a->eps, a->gate_first);
        PICOLM_LAUNCH_CHECK("gated_norm (wide)");
        return 0;
    }
    const int64_t blocks = ceil_div64(n_units, 4);
    if (v->dtype == PICOLM_F32)
        gated_norm_kernel<float><<<(unsigned)blocks, 4 * WAVE, 0, v->stream>>>((const float*)v->in, (const float*)v->extra[0], a->gate_stride,
                                                                               a->gate_off, (float*)v->out, a->weight, a->weight_len, a->width,
                                                                               a->group, a->eps, a->gate_first, n_units);
    else
        gated_norm_kernel<bf16_t><<<(unsigned)blocks, 4 * WAVE, 0, v->stream>>>((const float*)v->in, (const float*)v->extra[0], a->gate_stride,
                                                                                a->gate_off, (bf16_t*)v->out, a->weight, a->weight_len,
                                                                                a->width, a->group, a->eps, a->gate_first, n_units);
    PICOLM_LAUNCH_CHECK("gated_norm");
    return 0;
}

// ---- two normed branches meet the residual rows ------------------------------------------------------
__global__ __launch_bounds__(1024) void normed_sum_kernel(float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ b,
                                  const float* __restrict__ w_a, const float* __restrict__ w_b, int W, float eps, float mult) {
    __shared__ float scratch[16];
    const size_t row = blockIdx.x;
    const float* ar = a + row * W;
    const float* br = b ? b + row * W : nullptr;
    float sa = 0.f, sb = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        sa += ar[c] * ar[c];
        if (br) sb += br[c] * br[c];
    }
    sa = block_sum(sa, scratch);
    const float inv_a = 1.f / sqrtf(sa / (float)W + eps);
    float inv_b = 0.f;
    if (br) {
        sb = block_sum(sb, scratch);
        inv_b = 1.f / sqrtf(sb / (float)W + eps);
    }
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        float y = ar[c] * inv_a * w_a[c];
        if (br) y += br[c] * inv_b * w_b[c];
        x[row * W + c] += mult * y;
    }
}

extern "C" int picolm_call_normed_sum(void* user, const picolm_step_view* v) {
    const picolm_normed_sum_args* a = (const picolm_normed_sum_args*)user;
    VIEW_REQUIRE("normed_sum", v);
    PICOLM_REQUIRE(a && a->w_a && v->in && v->out && a->width > 0 && (!a->w_b) == (!v->extra[0]), "normed_sum: weights or buffers are missing");
    PICOLM_REQUIRE(v->in_row_bytes >= a->width * 4 && v->out_row_bytes >= a->width * 4 && (!v->extra[0] || v->extra_row_bytes[0] >= a->width * 4),
                   "normed_sum: rows too short for a width of %d", a->width);
    if (v->rows <= 0) return 0;
    normed_sum_kernel<<<v->rows, v->rows < 1024 && a->width >= 1024 ? 1024 : 256, 0, v->stream>>>((float*)v->out, (const float*)v->in, (const float*)v->extra[0], a->w_a, a->w_b, a->width,
                                                      a->eps, a->mult);
    PICOLM_LAUNCH_CHECK("normed_sum");
    return 0;
}

// ---- a function of every element ------------------------------------------------------------------------
template <typename TI, typename TO>
__global__ void map_rows_kernel(const TI* __restrict__ in, TO* __restrict__ out, int64_t n, int kind, float param) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const float x = to_f32<TI>(in[i]);
        float y = x;
        if (kind == 1) {
            const float p = fmaxf(x, 0.f);
            y = p * p;
        } else if (kind == 2) {
            y = param * tanhf(x / param);
        } else if (kind == 3) {
            y = param * x;
        }
        out[i] = from_f32<TO>(y);
    }
}

extern "C" int picolm_call_map_rows(void* user, const picolm_step_view* v) {
    const picolm_map_rows_args* a = (const picolm_map_rows_args*)user;
    VIEW_REQUIRE("map_rows", v);
    PICOLM_REQUIRE(a && v->out && a->width > 0 && (a->kind == 1 || (a->kind == 2 && a->param > 0.f) || a->kind == 3), "map_rows: kind %d over a width of %d",
                   a ? a->kind : -1, a ? a->width : 0);
    PICOLM_REQUIRE((a->in_dtype == PICOLM_F32 || a->in_dtype == PICOLM_BF16) && (a->out_dtype == PICOLM_F32 || a->out_dtype == PICOLM_BF16),
                   "map_rows: unknown dtype");
    PICOLM_REQUIRE(v->in || a->in_dtype == a->out_dtype, "map_rows: in place needs one dtype");
    PICOLM_REQUIRE(v->out_row_bytes >= a->width * elem_bytes(a->out_dtype) && (!v->in || v->in_row_bytes >= a->width * elem_bytes(a->in_dtype)),
                   "map_rows: rows too short for a width of %d", a->width);
    if (v->rows <= 0) return 0;
    const int64_t n = (int64_t)v->rows * a->width;
    const unsigned blocks = (unsigned)std::min<int64_t>(ceil_div64(n, 256), 65536);
    const void* in = v->in ? v->in : v->out;
    const bool fi = a->in_dtype == PICOLM_F32, fo = a->out_dtype == PICOLM_F32;
    if (fi && fo)
        map_rows_kernel<float, float><<<blocks, 256, 0, v->stream>>>((const float*)in, (float*)v->out, n, a->kind, a->param);
    else if (fi)
        map_rows_kernel<float, bf16_t><<<blocks, 256, 0, v->stream>>>((const float*)in, (bf16_t*)v->out, n, a->kind, a->param);
    else if (fo)
        map_rows_kernel<bf16_t, float><<<blocks, 256, 0, v->stream>>>((const bf16_t*)in, (float*)v->out, n, a->kind, a->param);
    else
        map_rows_kernel<bf16_t, bf16_t><<<blocks, 256, 0, v->stream>>>((const bf16_t*)in, (bf16_t*)v->out, n, a->kind, a->param);
    PICOLM_LAUNCH_CHECK("map_rows");
    return 0;
}
