// The steps either side of the expert GEMVs of a mixture-of-experts layer, on the device:
// router softmax + top-k, grouping of (token, slot) pairs by expert, the gated activation
// between the two projections, and the gate-weighted combine.
//
// Reference semantics:
//   route    moe.rs:466-486   logits -> f32, softmax over experts (linear.rs:160-171),
//                             arg_sort descending (stable: equal scores keep expert order),
//                             first top_k, optional renormalisation by their sum
//   group    moe.rs:563-590   dispatch_sparse: per expert the list of its tokens and gate
//                             weights, tokens ascending, slots in order
//   activate ffn_kernels.metal:19-242 gated SiLU / GeLU-tanh over [.., gate | up] (f32 math,
//                             one rounding) and moe.rs:152-173 GPT-OSS clamped SwiGLU over
//                             interleaved (gate, up) pairs
//   combine  moe.rs:592-605   output[token] += weight * expert_out[pair]
//
// The reference builds the lists on the host after copying the router output back and then
// launches one set of kernels per active expert; here nothing leaves the device, and the
// grouped expert GEMV consumes the lists directly (expert_offsets / token_ids).
// All of it is integer / small elementwise work bound by launch latency; every kernel is
// deterministic (no atomics on floats, fixed orders).

#include <cstdlib>

#include "oxq_device.hpp"
#include "oxq_internal.hpp"

namespace oxq {

template <typename T> __device__ __forceinline__ float load_f32(const T *p, size_t i);
template <> __device__ __forceinline__ float load_f32<float>(const float *p, size_t i) { return p[i]; }
struct F16Tag { uint16_t v; };
struct BF16Tag { uint16_t v; };
template <> __device__ __forceinline__ float load_f32<F16Tag>(const F16Tag *p, size_t i) {
    return F16Traits::to_f32(p[i].v);
}
template <> __device__ __forceinline__ float load_f32<BF16Tag>(const BF16Tag *p, size_t i) {
    return BF16Traits::to_f32(p[i].v);
}
template <typename T> __device__ __forceinline__ void store_f32(T *p, size_t i, float v);
template <> __device__ __forceinline__ void store_f32<float>(float *p, size_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void store_f32<F16Tag>(F16Tag *p, size_t i, float v) {
    p[i].v = F16Traits::from_f32(v);
}
template <> __device__ __forceinline__ void store_f32<BF16Tag>(BF16Tag *p, size_t i, float v) {
    p[i].v = BF16Traits::from_f32(v);
}

// ---------------------------------------------------------------------------
// route: one wave per token, probabilities in LDS
// ---------------------------------------------------------------------------
// one token, one wave: lane s < top_k ends with slot s in (my_idx, my_val); probs = E floats of LDS
template <typename T>
__device__ __forceinline__ void route_token(const T *__restrict__ l, int E, int top_k, int norm_topk, float *probs,
                                            int lane, int &out_idx, float &out_val) {
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, load_f32(l, e));
    mx = wave_all_reduce(mx, [](float a, float b) { return fmaxf(a, b); });
    float sum = 0.0f;
    for (int e = lane; e < E; e += 64) {
        const float p = expf(load_f32(l, e) - mx);
        probs[e] = p;
        sum += p;
    }
    sum = wave_all_reduce(sum, [](float a, float b) { return a + b; });
    for (int e = lane; e < E; e += 64) probs[e] = probs[e] / sum;
    // the wave's own LDS writes are visible to its own later reads (same wave, in order)
    float chosen_sum = 0.0f, my_val = 0.0f;
    int my_idx = 0;
    for (int s = 0; s < top_k; ++s) {
        float bv = -1.0f;
        int bi = 0x7fffffff;
        for (int e = lane; e < E; e += 64) {
            const float p = probs[e];
            if (p > bv) {  // strict: the lowest index wins among equals within a lane
                bv = p;
                bi = e;
            }
        }
        // the largest value, then the lowest index among the lanes that hold it
        const float best = wave_all_reduce(bv, [](float a, float b) { return fmaxf(a, b); });
        bi = wave_all_reduce(bv == best ? bi : 0x7fffffff, [](int a, int b) { return a < b ? a : b; });
        bv = best;
        if (bi >= E) {
            // Nothing compared greater: the probabilities are NaN (a NaN or +inf logit makes the whole row
            // NaN).  A stable sort leaves such a row in index order, so the slot takes the lowest index not
            // taken yet and its (NaN) value: top_idx always stays inside [0, E).
            int fi = 0x7fffffff;
            for (int e = lane; e < E; e += 64)
                if (!(probs[e] == -2.0f) && e < fi) fi = e;
            bi = wave_all_reduce(fi, [](int a, int b) { return a < b ? a : b; });
            bv = probs[bi < E ? bi : 0];
        }
        if (lane == s) {  // slot s is kept by lane s
            my_val = bv;
            my_idx = bi;
        }
        if (lane == 0 && bi < E) probs[bi] = -2.0f;  // taken
        chosen_sum += bv;  // slot order, as the reference's sum over the gathered values
    }
    out_idx = my_idx;
    out_val = norm_topk ? my_val / chosen_sum : my_val;
}

template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(const T *__restrict__ logits, int ntok, int E, int top_k,
                                                        int norm_topk, int32_t *__restrict__ top_idx,
                                                        float *__restrict__ top_vals) {
    extern __shared__ float route_lds[];  // [4 waves][E]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = blockIdx.x * 4 + wave;
    if (t >= ntok) return;  // wave-uniform; no barrier below
    int my_idx;
    float my_val;
    route_token(logits + (size_t)t * E, E, top_k, norm_topk, route_lds + (size_t)wave * E, lane, my_idx, my_val);
    if (lane < top_k) {
        const size_t i = (size_t)t * top_k + lane;
        top_idx[i] = my_idx;
        top_vals[i] = my_val;
    }
}

// The lanes of the wave that hold the same expert id as this lane (itself included), for lanes with
// `ok`: one ballot per bit of the id, no loop over experts.
__device__ __forceinline__ unsigned long long lanes_with_my_expert(int e, bool ok, int id_bits) {
    unsigned long long m = __ballot(ok);
    for (int j = 0; j < id_bits; ++j) {  // wave-uniform trip count
        const bool bit = (e >> j) & 1;
        const unsigned long long b = __ballot(ok && bit);
        m &= bit ? b : ~b;
    }
    return m;
}
__device__ __forceinline__ int expert_id_bits(int E) { return E > 1 ? 32 - __builtin_clz(E - 1) : 0; }

// Decode sizes (P <= 64), one wave: the pairs of (top_idx, top_vals) grouped by expert.  `scratch` = 2 E ints of LDS.
__device__ __forceinline__ void group_pairs_small(const int32_t *top_idx, const float *top_vals, int P, int E, int top_k,
                                                  int32_t *scratch, int lane, int32_t *__restrict__ offsets,
                                                  int32_t *__restrict__ tokens, float *__restrict__ weights,
                                                  int32_t *__restrict__ pair_pos) {
    // Decode sizes: one pair per lane, no counting matrix.  rank = the lanes below me with my expert
    // (pair order = token order inside an expert), count = all of them; the lowest such lane records it.
    int32_t *count = scratch;  // [E], then start[E]
    int32_t *start = scratch + E;
    for (int e = lane; e < E; e += 64) count[e] = 0;
    const int e = lane < P ? top_idx[lane] : -1;
    const bool ok = e >= 0 && e < E;  // ids outside [0, E) are dropped
    const unsigned long long mine = lanes_with_my_expert(e, ok, expert_id_bits(E));
    const int rank = __builtin_popcountll(mine & ((1ull << lane) - 1ull));
    if (ok && rank == 0) count[e] = __builtin_popcountll(mine);
    // exclusive scan of the counts in expert order, 64 experts per round
    int carry = 0;
    for (int e1 = 0; e1 < E; e1 += 64) {
        const int ee = e1 + lane;
        const int c = ee < E ? count[ee] : 0;
        int incl = c;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int t = __shfl_up(incl, off, 64);
            if (lane >= off) incl += t;
        }
        if (ee < E) {
            start[ee] = carry + incl - c;
            offsets[ee] = carry + incl - c;
        }
        carry += __shfl(incl, 63, 64);
    }
    if (lane == 0) offsets[E] = carry;
    if (ok) {
        const int pos = start[e] + rank;
        tokens[pos] = lane / top_k;
        weights[pos] = top_vals[lane];
        pair_pos[lane] = pos;
    }
}

// ---------------------------------------------------------------------------
// group.  Up to 64 pairs: one wave, one pair per lane (group_pairs_small).  Above: 16 waves, wave w
// owns the pairs [w C, (w + 1) C) and takes them 64 at a time, ranking the lanes that share an expert
// with ballots exactly as the small form does; its running count per expert lives in its own row of LDS,
// and the rank inside (wave, expert) is parked in pair_pos.  A scan over (expert, wave) then gives every
// wave its first position per expert, and a second pass over the pairs writes the lists.  Pair order
// inside an expert is pair order, whatever the scheduling: every sum here is over integers.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(64) void moe_group_kernel(const int32_t *__restrict__ top_idx,
                                                       const float *__restrict__ top_vals, int P, int E,
                                                       int32_t *__restrict__ offsets, int32_t *__restrict__ tokens,
                                                       float *__restrict__ weights, int32_t *__restrict__ pair_pos,
                                                       int top_k) {
    extern __shared__ int32_t group_lds[];  // count[E], start[E]
    group_pairs_small(top_idx, top_vals, P, E, top_k, group_lds, (int)threadIdx.x, offsets, tokens, weights, pair_pos);
}

constexpr int GROUP_WAVES = 16;
__global__ __launch_bounds__(GROUP_WAVES * 64) void moe_group_waves_kernel(
    const int32_t *__restrict__ top_idx, const float *__restrict__ top_vals, int P, int E,
    int32_t *__restrict__ offsets, int32_t *__restrict__ tokens, float *__restrict__ weights,
    int32_t *__restrict__ pair_pos, int top_k) {
    extern __shared__ int32_t group_lds[];  // cnt[GROUP_WAVES][E], then start[E]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int32_t *cnt = group_lds + (size_t)wave * E;
    int32_t *start = group_lds + (size_t)GROUP_WAVES * E;
    for (int e = lane; e < E; e += 64) cnt[e] = 0;  // the wave's own row: its LDS accesses stay in order
    const int C = ((P + GROUP_WAVES * 64 - 1) / (GROUP_WAVES * 64)) * 64;  // pairs per wave, whole batches of 64
    const int i0 = min(P, wave * C), i1 = min(P, i0 + C);
    const unsigned long long below = (1ull << lane) - 1ull;
    const int id_bits = expert_id_bits(E);
    for (int b = i0; b < i1; b += 64) {
        const int i = b + lane;
        const int e = i < i1 ? top_idx[i] : -1;
        const bool ok = e >= 0 && e < E;  // ids outside [0, E) are dropped
        const unsigned long long mine = lanes_with_my_expert(e, ok, id_bits);
        const int r = __builtin_popcountll(mine & below);
        const int before = ok ? cnt[e] : 0;  // every lane reads before the lowest lane of each expert adds
        if (ok && r == 0) cnt[e] = before + __builtin_popcountll(mine);
        const int rank = before + r;
        if (ok) pair_pos[i] = rank;  // within (wave, expert); made absolute below
    }
    __syncthreads();
    // per expert: exclusive prefix over the waves, total in start[e]
    for (int e = threadIdx.x; e < E; e += GROUP_WAVES * 64) {
        int c[GROUP_WAVES], run = 0;
#pragma unroll
        for (int w = 0; w < GROUP_WAVES; ++w) c[w] = group_lds[(size_t)w * E + e];  // independent reads first
#pragma unroll
        for (int w = 0; w < GROUP_WAVES; ++w) {
            group_lds[(size_t)w * E + e] = run;
            run += c[w];
        }
        start[e] = run;
    }
    __syncthreads();
    if (wave == 0) {  // exclusive scan of the totals in expert order, 64 experts per round
        int carry = 0;
        for (int e1 = 0; e1 < E; e1 += 64) {
            const int ee = e1 + lane;
            const int c = ee < E ? start[ee] : 0;
            int incl = c;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const int t = __shfl_up(incl, off, 64);
                if (lane >= off) incl += t;
            }
            if (ee < E) {
                start[ee] = carry + incl - c;
                offsets[ee] = carry + incl - c;
            }
            carry += __shfl(incl, 63, 64);
        }
        if (lane == 0) offsets[E] = carry;
    }
    __syncthreads();
    for (int b = i0; b < i1; b += 64) {
        const int i = b + lane;
        if (i >= i1) continue;
        const int e = top_idx[i];
        if (e < 0 || e >= E) continue;
        const int pos = start[e] + cnt[e] + pair_pos[i];
        tokens[pos] = i / top_k;
        weights[pos] = top_vals[i];
        pair_pos[i] = pos;
    }
}

// ---------------------------------------------------------------------------
// route + group in one launch for decode sizes (n_tokens * top_k <= 64): the waves route the tokens
// between them, the choices stay in LDS, and after one barrier wave 0 groups them.  Same arithmetic
// and the same outputs as the two kernels above, one launch period less.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(1024) void moe_route_group_kernel(const T *__restrict__ logits, int ntok, int E, int top_k,
                                                               int norm_topk, int32_t *__restrict__ top_idx,
                                                               float *__restrict__ top_vals, int32_t *__restrict__ offsets,
                                                               int32_t *__restrict__ tokens, float *__restrict__ weights,
                                                               int32_t *__restrict__ pair_pos) {
    extern __shared__ float rg_lds[];  // [waves][E] probabilities, [64] chosen experts, [64] their weights, [2 E] group scratch
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    int32_t *s_idx = (int32_t *)(rg_lds + (size_t)nw * E);
    float *s_val = (float *)(s_idx + 64);
    int32_t *scratch = (int32_t *)(s_val + 64);
    for (int t = wave; t < ntok; t += nw) {
        int my_idx;
        float my_val;
        route_token(logits + (size_t)t * E, E, top_k, norm_topk, rg_lds + (size_t)wave * E, lane, my_idx, my_val);
        if (lane < top_k) {
            const int i = t * top_k + lane;
            top_idx[i] = my_idx;
            top_vals[i] = my_val;
            s_idx[i] = my_idx;
            s_val[i] = my_val;
        }
    }
    __syncthreads();
    if (wave == 0)
        group_pairs_small(s_idx, s_val, ntok * top_k, E, top_k, scratch, lane, offsets, tokens, weights, pair_pos);
}

// ---------------------------------------------------------------------------
// gated activation
// ---------------------------------------------------------------------------

template <typename T, int KIND>
__global__ __launch_bounds__(256) void gated_act_kernel(const T *__restrict__ gu, T *__restrict__ out, size_t n_out,
                                                        int half_n, float limit) {
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= n_out) return;
    const size_t row = gid / half_n, col = gid % half_n;
    float r;
    if (KIND == OXQ_ACT_GPT_OSS_SWIGLU) {  // interleaved (gate, up), moe.rs:152-173
        r = gpt_oss_swiglu_f32(load_f32(gu, row * 2 * half_n + 2 * col), load_f32(gu, row * 2 * half_n + 2 * col + 1), limit);
    } else {  // [gate | up], ffn_kernels.metal:19-242
        const float g = load_f32(gu, row * 2 * half_n + col);
        const float u = load_f32(gu, row * 2 * half_n + half_n + col);
        r = mul_f32_rn(KIND == OXQ_ACT_GATED_SILU ? silu_f32(g) : gelu_tanh_f32(g), u);
    }
    store_f32(out, gid, r);
}

// 16-bit tensors with whole 16-byte pieces per row half: 8 outputs a thread ([gate | up]: one piece of each
// half; interleaved: two pieces of pairs), the same element functions as above.
template <typename TT, int KIND>
__global__ __launch_bounds__(256) void gated_act_vec_kernel(const uint16_t *__restrict__ gu, uint16_t *__restrict__ out,
                                                            size_t n_vec, int half_n, float limit) {
    const size_t vid = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (vid >= n_vec) return;
    const int vpr = half_n >> 3;  // vectors per output row
    const size_t row = vid / vpr;
    const int col = (int)(vid - row * vpr) * 8;
    const uint16_t *in = gu + row * 2 * (size_t)half_n;
    u32x4_t a, b;
    if (KIND == OXQ_ACT_GPT_OSS_SWIGLU) {
        a = *(const u32x4_t *)(in + 2 * col);
        b = *(const u32x4_t *)(in + 2 * col + 8);
    } else {
        a = *(const u32x4_t *)(in + col);
        b = *(const u32x4_t *)(in + half_n + col);
    }
    const uint32_t a0 = a[0], a1 = a[1], a2 = a[2], a3 = a[3], b0 = b[0], b1 = b[1], b2 = b[2], b3 = b[3];
    const uint32_t av[4] = {a0, a1, a2, a3}, bv[4] = {b0, b1, b2, b3};
    uint32_t o[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        float r[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if (KIND == OXQ_ACT_GPT_OSS_SWIGLU) {  // output 2q + h: pair (gate, up) = one 32-bit word
                const uint32_t w = (2 * q + h) < 4 ? av[2 * q + h] : bv[2 * q + h - 4];
                r[h] = gpt_oss_swiglu_f32(TT::to_f32((uint16_t)(w & 0xFFFFu)), TT::to_f32((uint16_t)(w >> 16)), limit);
            } else {
                const float g = TT::to_f32((uint16_t)(h ? av[q] >> 16 : av[q] & 0xFFFFu));
                const float u = TT::to_f32((uint16_t)(h ? bv[q] >> 16 : bv[q] & 0xFFFFu));
                r[h] = mul_f32_rn(KIND == OXQ_ACT_GATED_SILU ? silu_f32(g) : gelu_tanh_f32(g), u);
            }
        }
        o[q] = (uint32_t)TT::from_f32(r[0]) | ((uint32_t)TT::from_f32(r[1]) << 16);
    }
    *(u32x4_t *)(out + row * (size_t)half_n + col) = u32x4_t{o[0], o[1], o[2], o[3]};
}

// Two-tensor form (ffn_kernels.metal:72-110 silu_mul, 164-200 gelu_tanh_mul): the gate and the up
// projection are separate tensors of equal element count.
template <typename T, int KIND>
__global__ __launch_bounds__(256) void act_mul_kernel(const T *gate, const T *up, T *out, size_t n) {  // out may be gate
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= n) return;
    const float g = load_f32(gate, gid);
    const float a = KIND == OXQ_ACT_GATED_SILU ? silu_f32(g) : gelu_tanh_f32(g);
    // up == nullptr: the ungated FFN (ffn.rs:463-468), the activation alone
    store_f32(out, gid, up ? mul_f32_rn(a, load_f32(up, gid)) : a);
}

// ---------------------------------------------------------------------------
// combine: out[t] = sum over slots of w[t, s] * expert_out[pair_pos[t, s]] (f32, slot order)
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(const T *__restrict__ eo, const int32_t *__restrict__ pair_pos,
                                                          const float *__restrict__ top_vals, T *__restrict__ out,
                                                          int ntok, int H, int top_k) {
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (size_t)ntok * H) return;
    const int t = (int)(gid / H), h = (int)(gid % H);
    float acc = 0.0f;
    constexpr int MAXK = 8;
    if (top_k <= MAXK) {
        // all positions first, then all expert outputs, then the sum in slot order: two dependent loads deep
        // instead of two per slot
        int pos[MAXK];
        float w[MAXK], v[MAXK];
#pragma unroll
        for (int s = 0; s < MAXK; ++s)
            if (s < top_k) {
                pos[s] = pair_pos[(size_t)t * top_k + s];
                w[s] = top_vals[(size_t)t * top_k + s];
            }
#pragma unroll
        for (int s = 0; s < MAXK; ++s)
            if (s < top_k) v[s] = load_f32(eo, (size_t)pos[s] * H + h);
#pragma unroll
        for (int s = 0; s < MAXK; ++s)
            if (s < top_k) acc = fmaf(w[s], v[s], acc);
    } else {
        for (int s = 0; s < top_k; ++s) {
            const int pos = pair_pos[(size_t)t * top_k + s];
            acc = fmaf(top_vals[(size_t)t * top_k + s], load_f32(eo, (size_t)pos * H + h), acc);
        }
    }
    store_f32(out, gid, acc);
}

// The same sums eight columns a thread (16-bit types, H a multiple of 8, 16-byte aligned rows): one 16-byte load a
// slot and one 16-byte store instead of eight 2-byte ones each - at prefill sizes the scalar form moves 2 TB/s.
// Slot order and f32 arithmetic are the scalar kernel's: the same bits.
template <typename T>
__global__ __launch_bounds__(256) void moe_combine_vec_kernel(const T *__restrict__ eo, const int32_t *__restrict__ pair_pos,
                                                              const float *__restrict__ top_vals, T *__restrict__ out,
                                                              int ntok, int H8, int top_k) {
    const size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= (size_t)ntok * H8) return;
    const int t = (int)(gid / H8), h8 = (int)(gid % H8);
    constexpr int MAXK = 8;
    int pos[MAXK];
    float w[MAXK];
    u32x4_t v[MAXK];
#pragma unroll
    for (int s = 0; s < MAXK; ++s)
        if (s < top_k) {
            pos[s] = pair_pos[(size_t)t * top_k + s];
            w[s] = top_vals[(size_t)t * top_k + s];
        }
#pragma unroll
    for (int s = 0; s < MAXK; ++s)
        if (s < top_k) v[s] = *(const u32x4_t *)(eo + ((size_t)pos[s] * H8 + h8) * 8);
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < MAXK; ++s)
        if (s < top_k) {
            const T *e = (const T *)&v[s];
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] = fmaf(w[s], load_f32(e, (size_t)i), acc[i]);
        }
    u32x4_t o;
    T *op = (T *)&o;
#pragma unroll
    for (int i = 0; i < 8; ++i) store_f32(op, (size_t)i, acc[i]);
    *(u32x4_t *)(out + gid * 8) = o;
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------
int launch_moe_route(oxq_ctx *ctx, hipStream_t s, const void *logits, int dtype, int64_t T, int64_t E, int64_t top_k,
                     int norm_topk, int32_t *top_idx, float *top_vals) {
    dim3 grid((unsigned)ceil_div(T, 4)), block(256);
    set_plan(ctx, "moe_route", grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    const size_t lds = (size_t)4 * E * sizeof(float);
    if (dtype == OXQ_F32)
        hipLaunchKernelGGL(moe_route_kernel<float>, grid, block, lds, s, (const float *)logits, (int)T, (int)E,
                           (int)top_k, norm_topk, top_idx, top_vals);
    else if (dtype == OXQ_F16)
        hipLaunchKernelGGL(moe_route_kernel<F16Tag>, grid, block, lds, s, (const F16Tag *)logits, (int)T, (int)E,
                           (int)top_k, norm_topk, top_idx, top_vals);
    else
        hipLaunchKernelGGL(moe_route_kernel<BF16Tag>, grid, block, lds, s, (const BF16Tag *)logits, (int)T, (int)E,
                           (int)top_k, norm_topk, top_idx, top_vals);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

int launch_moe_group(oxq_ctx *ctx, hipStream_t s, const int32_t *top_idx, const float *top_vals, int64_t P, int64_t E,
                     int64_t top_k, int32_t *offsets, int32_t *tokens, float *weights, int32_t *pair_pos) {
    const bool small = P <= 64;
    dim3 grid(1), block(small ? 64 : GROUP_WAVES * 64);
    set_plan(ctx, "moe_group", grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    if (small) {
        hipLaunchKernelGGL(moe_group_kernel, grid, block, 2 * (size_t)E * sizeof(int32_t), s, top_idx, top_vals, (int)P,
                           (int)E, offsets, tokens, weights, pair_pos, (int)top_k);
    } else {
        const size_t lds = ((size_t)GROUP_WAVES + 1) * (size_t)E * sizeof(int32_t);  // at most 17 KB (256 experts)
        hipLaunchKernelGGL(moe_group_waves_kernel, grid, block, lds, s, top_idx, top_vals, (int)P, (int)E, offsets,
                           tokens, weights, pair_pos, (int)top_k);
    }
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

int launch_moe_route_group(oxq_ctx *ctx, hipStream_t s, const void *logits, int dtype, int64_t T, int64_t E,
                           int64_t top_k, int norm_topk, int32_t *top_idx, float *top_vals, int32_t *offsets,
                           int32_t *tokens, float *weights, int32_t *pair_pos) {
    const int nw = (int)std::min<int64_t>(T, 16);
    dim3 grid(1), block((unsigned)nw * 64);
    set_plan(ctx, "moe_route_group", grid, block, 1, 1, 0);
    if (ctx->plan_only) return OXQ_OK;
    const size_t lds = ((size_t)nw * E + 128 + 2 * (size_t)E) * sizeof(float);
#define OXQ_RG(TY)                                                                                                   \
    do {                                                                                                             \
        static LdsGrant lds_grant;                                                                                   \
        OXQ_HIP_CHECK(lds_grant.ensure((const void *)moe_route_group_kernel<TY>, lds));                              \
        hipLaunchKernelGGL(moe_route_group_kernel<TY>, grid, block, lds, s, (const TY *)logits, (int)T, (int)E,      \
                           (int)top_k, norm_topk, top_idx, top_vals, offsets, tokens, weights, pair_pos);            \
    } while (0)
    if (dtype == OXQ_F32) OXQ_RG(float);
    else if (dtype == OXQ_F16) OXQ_RG(F16Tag);
    else OXQ_RG(BF16Tag);
#undef OXQ_RG
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

template <typename T>
static void gated_go(hipStream_t s, dim3 grid, int kind, const void *gu, void *out, size_t n_out, int half_n,
                     float limit) {
    dim3 block(256);
    if (kind == OXQ_ACT_GATED_SILU)
        hipLaunchKernelGGL((gated_act_kernel<T, OXQ_ACT_GATED_SILU>), grid, block, 0, s, (const T *)gu, (T *)out, n_out,
                           half_n, limit);
    else if (kind == OXQ_ACT_GATED_GELU_TANH)
        hipLaunchKernelGGL((gated_act_kernel<T, OXQ_ACT_GATED_GELU_TANH>), grid, block, 0, s, (const T *)gu, (T *)out,
                           n_out, half_n, limit);
    else
        hipLaunchKernelGGL((gated_act_kernel<T, OXQ_ACT_GPT_OSS_SWIGLU>), grid, block, 0, s, (const T *)gu, (T *)out,
                           n_out, half_n, limit);
}

int launch_gated_activation(oxq_ctx *ctx, hipStream_t s, const void *gu, void *out, int dtype, int64_t rows,
                            int64_t half_n, int kind, float limit) {
    const size_t n_out = (size_t)rows * (size_t)half_n;
    dim3 grid((unsigned)ceil_div((int64_t)n_out, 256)), block(256);
    set_plan(ctx, kind == OXQ_ACT_GATED_SILU ? "gated_silu" : kind == OXQ_ACT_GATED_GELU_TANH ? "gated_gelu_tanh"
                                                                                             : "gpt_oss_swiglu",
             grid, block, 1, 1, 0);
    if (ctx->plan_only || n_out == 0) return OXQ_OK;
    // from 64 K vectors on (two workgroups a CU): below, one output a thread spreads the work wider and
    // is faster (decode: 2.0 against 2.5 us; 2048 x 2880 outputs: 13.1 against 10.2 us)
    const size_t vec_min = (size_t)std::max(0, tune(ctx, OXQ_TUNE_ACT_VEC, 65536));
    if (dtype != OXQ_F32 && half_n % 8 == 0 && (((uintptr_t)gu | (uintptr_t)out) & 15) == 0 && n_out / 8 >= vec_min) {
        const size_t n_vec = n_out / 8;
        dim3 vgrid((unsigned)ceil_div((int64_t)n_vec, 256));
#define OXQ_GV(TT, K)                                                                                                   \
    hipLaunchKernelGGL((gated_act_vec_kernel<TT, K>), vgrid, block, 0, s, (const uint16_t *)gu, (uint16_t *)out, n_vec, \
                       (int)half_n, limit)
        if (dtype == OXQ_F16) {
            if (kind == OXQ_ACT_GATED_SILU) OXQ_GV(F16Traits, OXQ_ACT_GATED_SILU);
            else if (kind == OXQ_ACT_GATED_GELU_TANH) OXQ_GV(F16Traits, OXQ_ACT_GATED_GELU_TANH);
            else OXQ_GV(F16Traits, OXQ_ACT_GPT_OSS_SWIGLU);
        } else {
            if (kind == OXQ_ACT_GATED_SILU) OXQ_GV(BF16Traits, OXQ_ACT_GATED_SILU);
            else if (kind == OXQ_ACT_GATED_GELU_TANH) OXQ_GV(BF16Traits, OXQ_ACT_GATED_GELU_TANH);
            else OXQ_GV(BF16Traits, OXQ_ACT_GPT_OSS_SWIGLU);
        }
#undef OXQ_GV
        OXQ_HIP_CHECK(hipGetLastError());
        return OXQ_OK;
    }
    if (dtype == OXQ_F32) gated_go<float>(s, grid, kind, gu, out, n_out, (int)half_n, limit);
    else if (dtype == OXQ_F16) gated_go<F16Tag>(s, grid, kind, gu, out, n_out, (int)half_n, limit);
    else gated_go<BF16Tag>(s, grid, kind, gu, out, n_out, (int)half_n, limit);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

template <typename T>
static void act_mul_go(hipStream_t s, dim3 grid, int kind, const void *gate, const void *up, void *out, size_t n) {
    dim3 block(256);
    if (kind == OXQ_ACT_GATED_SILU)
        hipLaunchKernelGGL((act_mul_kernel<T, OXQ_ACT_GATED_SILU>), grid, block, 0, s, (const T *)gate, (const T *)up,
                           (T *)out, n);
    else
        hipLaunchKernelGGL((act_mul_kernel<T, OXQ_ACT_GATED_GELU_TANH>), grid, block, 0, s, (const T *)gate,
                           (const T *)up, (T *)out, n);
}

int launch_activation_mul(oxq_ctx *ctx, hipStream_t s, const void *gate, const void *up, void *out, int dtype,
                          int64_t n, int kind) {
    dim3 grid((unsigned)ceil_div(n, 256)), block(256);
    set_plan(ctx, kind == OXQ_ACT_GATED_SILU ? (up ? "silu_mul" : "silu") : (up ? "gelu_tanh_mul" : "gelu_tanh"), grid,
             block, 1, 1, 0);
    if (ctx->plan_only || n == 0) return OXQ_OK;
    if (dtype == OXQ_F32) act_mul_go<float>(s, grid, kind, gate, up, out, (size_t)n);
    else if (dtype == OXQ_F16) act_mul_go<F16Tag>(s, grid, kind, gate, up, out, (size_t)n);
    else act_mul_go<BF16Tag>(s, grid, kind, gate, up, out, (size_t)n);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

int launch_moe_combine(oxq_ctx *ctx, hipStream_t s, const void *eo, const int32_t *pair_pos, const float *top_vals,
                       void *out, int dtype, int64_t T, int64_t H, int64_t top_k) {
    const size_t n = (size_t)T * (size_t)H;
    // eight columns a thread where the shape allows and the launch has the threads to spare
    const bool vec = dtype != OXQ_F32 && H % 8 == 0 && top_k <= 8 && n >= (size_t)1 << 19 &&
                     (ctx->plan_only || ((((uintptr_t)eo | (uintptr_t)out) & 15) == 0));
    dim3 grid((unsigned)ceil_div((int64_t)(vec ? n / 8 : n), 256)), block(256);
    set_plan(ctx, vec ? "moe_combine_x8" : "moe_combine", grid, block, 1, 1, 0);
    if (ctx->plan_only || n == 0) return OXQ_OK;
    if (vec) {
        if (dtype == OXQ_F16)
            hipLaunchKernelGGL(moe_combine_vec_kernel<F16Tag>, grid, block, 0, s, (const F16Tag *)eo, pair_pos, top_vals,
                               (F16Tag *)out, (int)T, (int)(H / 8), (int)top_k);
        else
            hipLaunchKernelGGL(moe_combine_vec_kernel<BF16Tag>, grid, block, 0, s, (const BF16Tag *)eo, pair_pos, top_vals,
                               (BF16Tag *)out, (int)T, (int)(H / 8), (int)top_k);
        OXQ_HIP_CHECK(hipGetLastError());
        return OXQ_OK;
    }
    if (dtype == OXQ_F32)
        hipLaunchKernelGGL(moe_combine_kernel<float>, grid, block, 0, s, (const float *)eo, pair_pos, top_vals,
                           (float *)out, (int)T, (int)H, (int)top_k);
    else if (dtype == OXQ_F16)
        hipLaunchKernelGGL(moe_combine_kernel<F16Tag>, grid, block, 0, s, (const F16Tag *)eo, pair_pos, top_vals,
                           (F16Tag *)out, (int)T, (int)H, (int)top_k);
    else
        hipLaunchKernelGGL(moe_combine_kernel<BF16Tag>, grid, block, 0, s, (const BF16Tag *)eo, pair_pos, top_vals,
                           (BF16Tag *)out, (int)T, (int)H, (int)top_k);
    OXQ_HIP_CHECK(hipGetLastError());
    return OXQ_OK;
}

}  // namespace oxq
