// bf16 softmax attention on the matrix cores over pages that the caller keeps in the order of the
// MFMA operands (attention.h: k_page_offset(key, i, d, true), v_page_offset(i, key, dv, true)), with what the vector-ALU kernels of attention_generic.hip take beside keys and
// values: values of a size of their own, a window, a bias by distance, a sink and an output gate.  Head sizes
// of 64, 96 and 128 on either side.
//
// A workgroup of PLAIN_WAVES waves per piece of work; the waves take the tiles of 32 keys in turn and
// add their results up through LDS at the end.  S^T = K Q^T and O^T = V^T P^T with 32x32x16 MFMAs as in
// attention_mfma.hip (a lane of the accumulator holds one query and 16 keys, so the softmax's
// maximum and sum are in-lane plus one exchange with lane ^ 32, and P^T feeds the second product
// from registers).  (Pages as plain arrays were measured first: a lane's 16 bytes of a key's row
// lie in a cache line of their own, a tile cost a thousand line look-ups in the CU's cache, and a
// tile took 8 us.)
//   prefill: a workgroup takes 32 new tokens (the step's tiles of 32 rows): of four query heads of one
//            KV group where the group has a multiple of four, a head a wave, so that the waves read
//            the same keys and values at about the same time and three of them find them in the
//            CU's cache; else of one head, whose keys the waves take in turn, 32 at a time; a wave's next tile's operands are asked for before
//            this tile's products, and the page after that is looked up in the page table.
//   decode : a workgroup takes one entry of the step's work list and one KV group; its columns are
//            the group's query heads (32 at a time).  A sequence of several chunks leaves partial
//            results for the merge kernel of attention_generic.hip.
// Statistics are float in the base-2 domain; the bias table is [H][bias_rows].
#include "common.h"
#include "api.h"
#include "attention.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

#define LOG2E 1.4426950408889634f
#define LN2 0.6931471805599453f

__device__ __forceinline__ bf16x8 ldg8(const bf16_t* p) { return *(const bf16x8*)p; }
__device__ __forceinline__ int key_of_elem(int e, int h) { return 16 * (e >> 3) + 8 * h + (e & 7); }
__device__ __forceinline__ float exp2_flushing(float x) { return __builtin_amdgcn_exp2f(x); }

template <int D, int DV>
struct TileOperands {
    bf16x8 K[D / 16];
    bf16x8 V[DV / 32][2];
};

// operands of the 32 keys from key `half * 32` of a page on: the pages are in the order of the
// operands (k_page_offset, v_page_offset of attention.h, the values' rows counted by DV), so that a
// wave's load of a chunk reads 1 KB in a row
template <int D, int DV>
__device__ __forceinline__ void load_tile(TileOperands<D, DV>& t, const bf16_t* kpage, const bf16_t* vpage, int half, int lane) {
    const bf16_t* kp = kpage + ((size_t)half * (D / 16) * 64 + lane) * 8;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) t.K[s] = ldg8(kp + 512 * s);
    const bf16_t* vp = vpage + ((size_t)half * (DV / 32) * 2 * 64 + lane) * 8;
#pragma unroll
    for (int dt = 0; dt < DV / 32; ++dt)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) t.V[dt][ks] = ldg8(vp + 512 * (2 * dt + ks));
}

#define PLAIN_WAVES 4

template <int D, int DV>
__global__ __launch_bounds__(64 * PLAIN_WAVES) void attn_plain_mfma_kernel(AttnArgs a) {
    extern __shared__ float merge_lds[];        // [PLAIN_WAVES - 1][DV / 2 + 2][64]: O^T, maximum and sum of the other waves
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, col = lane & 31, h = lane >> 5;
    const int R = a.H / a.G;
    int seq, g, head, tok, qpos, qpos_first, slot, page_lo, page_hi, hi, split = 0, n_chunks = 1;
    bool q_ok;
    if (a.decode) {
        DecodeWork w;
        int which;
        const int hc = (R + 31) / 32;
        if (!decode_work(a, a.G * hc, w, which)) return;
        seq = w.seq, split = w.split, n_chunks = w.n_chunks, slot = w.slot;
        g = which / hc;
        const int j = (which % hc) * 32 + col;
        q_ok = j < R;
        head = g * R + min(j, R - 1);
        tok = seq, qpos = qpos_first = w.qpos, hi = w.qpos;
        page_lo = w.page_lo, page_hi = w.page_hi;
    } else {
        seq = a.tile_seq[blockIdx.x];
        const int q0 = a.tile_q0[blockIdx.x], nnew = a.seq_nnew[seq], pos0 = a.seq_pos0[seq];
        head = a.waves_take_heads ? blockIdx.y * PLAIN_WAVES + wave : blockIdx.y;
        g = head / R;
        q_ok = q0 + col < nnew;
        const int l = min(q0 + col, nnew - 1);
        tok = a.cu_seqlens[seq] + l, qpos = pos0 + l, qpos_first = pos0 + q0;
        slot = a.seq_slot[seq];
        hi = pos0 + min(q0 + 31, nnew - 1);
        page_lo = first_seen(a, qpos_first) / PAGE_TOKENS, page_hi = hi / PAGE_TOKENS + 1;      // (the tile's first query sees furthest back)
    }
    // the wave's queries as operands: column `col`, k-step s covers elements 16 s + 8 h .. + 8
    bf16x8 Qf[D / 16];
    {
        const bf16_t* qp = (const bf16_t*)a.q + (size_t)tok * a.H * D + (size_t)head * D + 8 * h;
#pragma unroll
        for (int s = 0; s < D / 16; ++s) Qf[s] = ldg8(qp + 16 * s);
    }
    f32x16 O[DV / 32];
#pragma unroll
    for (int dt = 0; dt < DV / 32; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) O[dt][e] = 0.f;
    float m_run = NEG_BIG, l_run = 0.f;
    const float scale2 = a.scale * LOG2E;
    const float* bias = a.bias ? a.bias + (size_t)head * a.bias_rows : nullptr;
    const int last_row = a.bias_rows - 1;
    // (qpos_first is the wave's query nearest to the keys: a tile beyond the table's reach from there has one bias)

    const int32_t* pt = a.page_table + (size_t)slot * a.max_pages;
    const bf16_t* kbase = (const bf16_t*)a.k_pages + (size_t)g * PAGE_TOKENS * D;
    const bf16_t* vbase = (const bf16_t*)a.v_pages + (size_t)g * PAGE_TOKENS * DV;
    const size_t k_page_elems = (size_t)a.G * PAGE_TOKENS * D, v_page_elems = (size_t)a.G * PAGE_TOKENS * DV;

    const int tile_hi = min(2 * page_hi, hi / 32 + 1);       // tiles of 32 keys: this wave takes tile_lo, tile_lo + PLAIN_WAVES, ... below tile_hi
    const bool keys_in_turn = !a.waves_take_heads;           // the waves share one head's keys
    const int tile_step = keys_in_turn ? PLAIN_WAVES : 1;
    // with a window or stretches, the tile of 32 keys that holds the oldest key any query of this wave sees
    const int oldest = first_seen(a, qpos_first), my_oldest = first_seen(a, qpos);
    const int tile_lo = max(2 * page_lo, oldest / 32) + (keys_in_turn ? wave : 0);
    // two sets of operands in turn: the loads of the tile after this one are queued before this
    // tile's products and stay there (the scheduler may not move them past the barrier), and the
    // page of the tile after that is looked up meanwhile
    TileOperands<D, DV> A, B;
    auto fetch = [&](TileOperands<D, DV>& ops, int t, int phys) {
        load_tile<D, DV>(ops, kbase + (size_t)phys * k_page_elems, vbase + (size_t)phys * v_page_elems, t & 1, lane);
    };
    auto page_of = [&](int t) { return t < tile_hi ? pt[(t / 2) % a.ring_pages] : 0; };
    // a tile's 16 biases of a lane, in base-2 units: asked for before the next tile's operands, because
    // loads come back in the order they were queued and the softmax must not wait for those too
    auto load_bias = [&](int t, float (&bv)[16]) {
        const int key0 = 32 * t;
        if (!bias || t >= tile_hi) {
#pragma unroll
            for (int e = 0; e < 16; ++e) bv[e] = 0.f;
        } else if (qpos_first - (key0 + 31) >= last_row) {      // wave-uniform: every pair of the tile is beyond the table
            const float far_bias = bias[last_row] * LOG2E;
#pragma unroll
            for (int e = 0; e < 16; ++e) bv[e] = far_bias;
        } else {
#pragma unroll
            for (int e = 0; e < 16; ++e) bv[e] = bias[min(max(qpos - (key0 + key_of_elem(e, h)), 0), last_row)] * LOG2E;
        }
    };
    auto attend = [&](const TileOperands<D, DV>& ops, int t, const float (&bv)[16]) {
        const int key0 = 32 * t;
        f32x16 S;
#pragma unroll
        for (int e = 0; e < 16; ++e) S[e] = 0.f;
#pragma unroll
        for (int s = 0; s < D / 16; ++s) S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ops.K[s], Qf[s], S, 0, 0, 0);
        float mx = NEG_BIG;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int key = key0 + key_of_elem(e, h);
            const bool vis = q_ok && key <= qpos && key >= my_oldest;
            S[e] = vis ? fmaf(S[e], scale2, bv[e]) : NEG_BIG;
            mx = fmaxf(mx, S[e]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
        const float m_new = fmaxf(m_run, mx);
        const float alpha = exp2_flushing(m_run - m_new);
        float sum = 0.f;
        bf16x8 Pf[2];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const float p = S[e] > 0.5f * NEG_BIG ? exp2_flushing(S[e] - m_new) : 0.f;
            sum += p;
            Pf[e / 8][e % 8] = (__bf16)p;
        }
        sum += __shfl_xor(sum, 32, WAVE);
        l_run = l_run * alpha + sum;
        m_run = m_new;
#pragma unroll
        for (int dt = 0; dt < DV / 32; ++dt) {
#pragma unroll
            for (int e = 0; e < 16; ++e) O[dt][e] *= alpha;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ops.V[dt][ks], Pf[ks], O[dt], 0, 0, 0);
        }
    };
    if (tile_lo < tile_hi) fetch(A, tile_lo, page_of(tile_lo));
    int phys_b = page_of(tile_lo + tile_step), phys_a = 0;
    float bv[16];
    for (int t = tile_lo; t < tile_hi; t += 2 * tile_step) {
        const int tb = t + tile_step, ta = t + 2 * tile_step;
        load_bias(t, bv);
        __builtin_amdgcn_sched_barrier(0);
        if (tb < tile_hi) fetch(B, tb, phys_b);
        phys_a = page_of(ta);
        __builtin_amdgcn_sched_barrier(0);
        attend(A, t, bv);
        if (tb >= tile_hi) break;
        load_bias(tb, bv);
        __builtin_amdgcn_sched_barrier(0);
        if (ta < tile_hi) fetch(A, ta, phys_a);
        phys_b = page_of(ta + tile_step);
        __builtin_amdgcn_sched_barrier(0);
        attend(B, tb, bv);
    }
    // the other waves' results join the first wave's
    if (PLAIN_WAVES > 1 && keys_in_turn) {
        constexpr int PER = DV / 2 + 2;          // floats a lane leaves
        if (wave > 0) {
            float* mine = merge_lds + (size_t)(wave - 1) * PER * 64 + lane;
            mine[0] = m_run;
            mine[64] = l_run;
#pragma unroll
            for (int dt = 0; dt < DV / 32; ++dt)
#pragma unroll
                for (int e = 0; e < 16; ++e) mine[(2 + 16 * dt + e) * 64] = O[dt][e];
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int w = 0; w < PLAIN_WAVES - 1; ++w) {
            const float* other = merge_lds + (size_t)w * PER * 64 + lane;
            const float m_o = other[0], l_o = other[64];
            const float m_new = fmaxf(m_run, m_o);
            const float mine_k = exp2_flushing(m_run - m_new), other_k = exp2_flushing(m_o - m_new);
            l_run = l_run * mine_k + l_o * other_k;
            m_run = m_new;
#pragma unroll
            for (int dt = 0; dt < DV / 32; ++dt)
#pragma unroll
                for (int e = 0; e < 16; ++e) O[dt][e] = O[dt][e] * mine_k + other[(2 + 16 * dt + e) * 64] * other_k;
        }
    }
    if (!q_ok) return;
    // element 4 a + b of O[dt] is value column 32 dt + 8 a + 4 h + b of query `col`
    if (a.decode && n_chunks > 1) {
        float* po = a.partial + (((size_t)seq * a.H + head) * a.max_splits + split) * (DV + 2);
        if (h == 0) {
            po[0] = m_run > 0.5f * NEG_BIG ? m_run * LN2 : NEG_BIG;      // the merge works with e-based exponents
            po[1] = l_run;
        }
#pragma unroll
        for (int dt = 0; dt < DV / 32; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) po[2 + 32 * dt + 8 * (e >> 2) + 4 * h + (e & 3)] = O[dt][e];
        return;
    }
    float keep = 1.f;
    if (a.sink) {                   // one more term of the denominator, under a maximum that covers it
        const float s2 = a.sink[head] * LOG2E, top = fmaxf(m_run, s2);
        keep = exp2_flushing(m_run - top);
        l_run = l_run * keep + exp2_flushing(s2 - top);
    }
    const float inv = l_run > 0.f ? keep / l_run : 0.f;
    const size_t at = (size_t)tok * a.H * DV + (size_t)head * DV;
    const float* gate = a.gate ? a.gate + (size_t)tok * a.gate_stride + (size_t)head * DV : nullptr;
#pragma unroll
    for (int dt = 0; dt < DV / 32; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int c = 32 * dt + 8 * (e >> 2) + 4 * h + (e & 3);
            float y = O[dt][e] * inv;
            if (gate) y *= 1.f / (1.f + __expf(-gate[c]));
            if (a.out_float) ((float*)a.out)[at + c] = y;
            else ((bf16_t*)a.out)[at + c] = from_f32<bf16_t>(y);
        }
}

extern "C" int picolm_attn_plain_mfma_takes(int d, int dv) {
    return (d == 64 || d == 96 || d == 128) && (dv == 64 || dv == 96 || dv == 128) ? 1 : 0;
}
extern "C" int picolm_attn_plain_mfma_tile_rows(void) { return 32; }

template <int D>
static int launch_dv(const AttnArgs& a, int dv, dim3 grid, hipStream_t stream) {
    const size_t lds = sizeof(float) * (PLAIN_WAVES - 1) * (dv / 2 + 2) * 64;       // at most 50 KB
    if (dv == 64) attn_plain_mfma_kernel<D, 64><<<grid, 64 * PLAIN_WAVES, lds, stream>>>(a);
    else if (dv == 96) attn_plain_mfma_kernel<D, 96><<<grid, 64 * PLAIN_WAVES, lds, stream>>>(a);
    else attn_plain_mfma_kernel<D, 128><<<grid, 64 * PLAIN_WAVES, lds, stream>>>(a);
    PICOLM_LAUNCH_CHECK("attn_plain_mfma");
    return 0;
}
static int launch(const AttnArgs& a, int dv, dim3 grid, hipStream_t stream) {
    return a.d == 64 ? launch_dv<64>(a, dv, grid, stream) : a.d == 96 ? launch_dv<96>(a, dv, grid, stream) : launch_dv<128>(a, dv, grid, stream);
}

int check_attn_sizes(const char* who, int H, int G, int d, int max_pages, int ring_pages);
int check_decode_chunks(const char* who, const float* partial, const int32_t* chunk_list, int n_chunks, int pages_per_chunk, int max_splits);
int picolm_attn_merge_launch(const AttnArgs& a, int dt, int n_seq, hipStream_t stream);

static int fill_extras(const char* who, AttnArgs& a, const picolm_attn_extras* x, int& dv) {
    dv = x && x->v_head_dim > 0 ? x->v_head_dim : a.d;
    PICOLM_REQUIRE(picolm_attn_plain_mfma_takes(a.d, dv), "%s: keys of %d and values of %d are not sizes of the matrix-core kernel", who, a.d, dv);
    a.dv = dv == a.d ? 0 : dv;
    if (!x) return 0;
    PICOLM_REQUIRE(!x->bias || x->bias_rows >= 1, "%s: a bias by distance needs at least one row", who);
    PICOLM_REQUIRE(!x->gate || x->gate_stride >= a.H * dv, "%s: gate rows of %d floats for %d heads of %d", who, x->gate_stride, a.H, dv);
    PICOLM_REQUIRE(x->mask_window >= 0 && (a.window <= 0 || x->mask_window <= a.window), "%s: a window of %d keys over pages laid out for %d", who,
                   x->mask_window, a.window);
    a.bias = x->bias, a.bias_rows = x->bias_rows, a.sink = x->sink, a.gate = x->gate, a.gate_stride = x->gate_stride;
    a.mask_window = x->mask_window;
    PICOLM_REQUIRE(x->mask_chunk >= 0, "%s: stretches of %d keys", who, x->mask_chunk);
    a.mask_chunk = x->mask_chunk, a.out_float = x->out_float;
    return 0;
}

// tiles of picolm_attn_plain_mfma_tile_rows() rows; bfloat16 only
extern "C" int picolm_attn_prefill_plain_mfma(const void* q, const void* k_pages, const void* v_pages, void* out, const int32_t* tile_seq,
                                              const int32_t* tile_q0, int n_tiles, const int32_t* seq_slot, const int32_t* seq_pos0,
                                              const int32_t* seq_nnew, const int32_t* cu_seqlens, const int32_t* page_table, int max_pages,
                                              int ring_pages, int H, int G, int d, int window, float scale, const picolm_attn_extras* x,
                                              hipStream_t stream) {
    if (check_attn_sizes("attn_prefill_plain_mfma", H, G, d, max_pages, ring_pages)) return -1;
    PICOLM_REQUIRE(window >= 0, "attn_prefill_plain_mfma: a window of %d keys", window);
    PICOLM_REQUIRE(H <= 65535, "attn_prefill_plain_mfma: %d heads exceed the grid", H);
    if (n_tiles <= 0) return 0;
    AttnArgs a = {q, k_pages, v_pages, out, nullptr, tile_seq, tile_q0, seq_slot, seq_pos0, seq_nnew,
                  cu_seqlens, page_table, max_pages, ring_pages, H, G, d, window, scale, 0, nullptr, 0, 1,
                  nullptr, nullptr, nullptr, nullptr, 0};
    int dv;
    if (fill_extras("attn_prefill_plain_mfma", a, x, dv)) return -1;
    // (measured at 2,048 tokens: a head a wave is faster once its workgroups fill the 256 CUs, 0.39 against 0.47 ms
    // for two layers of 16 heads; with 8 heads the keys in turn are, 0.40 against 0.57 ms)
    a.waves_take_heads = (H / G) % PLAIN_WAVES == 0 && (int64_t)n_tiles * (H / PLAIN_WAVES) >= 256;
    return launch(a, dv, dim3(n_tiles, a.waves_take_heads ? H / PLAIN_WAVES : H), stream);
}

extern "C" int picolm_attn_decode_plain_mfma(const void* q, const void* k_pages, const void* v_pages, void* out, float* partial, int n_seq,
                                             const int32_t* chunk_list, int n_chunks, int pages_per_chunk, int max_splits,
                                             const int32_t* seq_pos0, const int32_t* page_table, int max_pages, int ring_pages, int H,
                                             int G, int d, int window, float scale, const picolm_attn_extras* x, hipStream_t stream) {
    if (check_attn_sizes("attn_decode_plain_mfma", H, G, d, max_pages, ring_pages)) return -1;
    PICOLM_REQUIRE(window >= 0, "attn_decode_plain_mfma: a window of %d keys", window);
    if (check_decode_chunks("attn_decode_plain_mfma", partial, chunk_list, n_chunks, pages_per_chunk, max_splits)) return -1;
    if (n_seq <= 0 || n_chunks <= 0) return 0;
    const int hc = ceil_div(H / G, 32);
    PICOLM_REQUIRE((int64_t)n_chunks * G * hc < (1ll << 31), "attn_decode_plain_mfma: %d chunks of %d waves exceed the grid", n_chunks, G * hc);
    AttnArgs a = {q, k_pages, v_pages, out, partial, nullptr, nullptr, nullptr, seq_pos0, nullptr, nullptr,
                  page_table, max_pages, ring_pages, H, G, d, window, scale, 1, chunk_list, pages_per_chunk, max_splits,
                  nullptr, nullptr, nullptr, nullptr, 0};
    int dv;
    if (fill_extras("attn_decode_plain_mfma", a, x, dv)) return -1;
    const int rc = launch(a, dv, dim3(n_chunks * G * hc), stream);
    if (rc) return rc;
    return max_splits > 1 ? picolm_attn_merge_launch(a, PICOLM_BF16, n_seq, stream) : 0;
}
