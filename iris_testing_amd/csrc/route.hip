// Router: logits = x @ W_r (+ bias) with a pinned fp32 reduction order, then softmax gates
// and top-k with wavefront-level reductions.
//
// Replaces the device work of `F.softmax(torch.einsum('th,he->te', tokens, router), dim=-1)`
// followed by `torch.topk(..., topk)` in the reference (utils.py:200-202).
//
// Reduction order (what makes the indices reproducible bit-for-bit on a CPU):
//   logit[t,e] = bias[e] + chain,  chain = fmaf(x[t,h], w[h,e], chain) for h = 0..H-1, chain0 = +0.0f
// Every (t,e) chain is one accumulator element walked over H in ascending order, so no cross-lane or
// cross-block partial sums exist.  The chains run on the matrix cores, but only through K = 1 fp32 MFMAs,
// which perform exactly one fused multiply-add per output element and instruction; MFMAs with K > 1 (and all
// bf16 ones) sum several products in an order that is not specified and are not used.
#include "common.h"
#include <type_traits>

namespace {

constexpr int RT_TB = 64;  // tokens per block: one per lane

template <typename XT>
struct VecLoad;
template <>
struct VecLoad<bf16_t> {
    static constexpr int N = 8;
    __device__ static void load(const bf16_t* p, float* out) { unpack(*reinterpret_cast<const uint4*>(p), out); }
    __device__ static void unpack(const uint4& v, float* out) {
        uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            out[2 * i] = __uint_as_float(w[i] << 16);
            out[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
};
template <>
struct VecLoad<float> {
    static constexpr int N = 4;
    __device__ static void load(const float* p, float* out) { unpack(*reinterpret_cast<const uint4*>(p), out); }
    __device__ static void unpack(const uint4& v, float* out) {
        out[0] = __uint_as_float(v.x); out[1] = __uint_as_float(v.y); out[2] = __uint_as_float(v.z); out[3] = __uint_as_float(v.w);
    }
};

// ---- logits on the matrix cores, still one fused multiply-add per (t, e, h) in ascending h -------------
// A K = 1 fp32 MFMA (v_mfma_f32_16x16x1_4b_f32, v_mfma_f32_4x4x1_16b_f32) performs, for every output element,
// exactly one D = fma(a, b, C) with a single rounding -- the same operation, bit for bit (subnormals
// included), as a v_fma_f32 or the fmaf of a CPU (checked on the GPU against fmaf chains over normal, wide-range,
// subnormal and bf16-valued operands); it runs the chains of 64 tokens x SHAPE experts in one instruction, at
// up to twice the vector rate, and takes its operands from two registers instead of 64 x SHAPE LDS reads.
//   A operand: lane l holds x[t0 + l][h]                 (lane = token: the wave's 64 tokens)
//   B operand: lane l holds w[h][e0 + l % SHAPE]         (the SHAPE experts, repeated across the lanes)
//   D, SHAPE = 16: register v holds token t0 + 16 * (v / 4) + 4 * (l / 16) + v % 4, expert e0 + l % 16
//   D, SHAPE = 4:  register v holds token t0 + 4 * (l / 4) + v,                     expert e0 + l % 4
// Block = NWV waves on the same 64 tokens, wave i on experts [e0 + i * SHAPE, + SHAPE).  Both operands are converted
// to fp32 on their way into LDS (the lane reads four consecutive h of its own token row, and of its expert in the
// transposed router slab, with one 128-bit read each).
typedef float rt_f4 __attribute__((ext_vector_type(4)));
typedef float rt_f16 __attribute__((ext_vector_type(16)));
typedef unsigned int rt_u4 __attribute__((ext_vector_type(4)));

template <typename XT, int SHAPE, int NWV>
__global__ __launch_bounds__(NWV * WAVE) void route_logits_mfma_kernel(const XT* __restrict__ x, const XT* __restrict__ w,
                                                                        const float* __restrict__ bias,
                                                                        float* __restrict__ logits, int T, int H, int E) {
    static_assert(SHAPE == 4 || SHAPE == 16, "experts per MFMA");
    constexpr int NTH = NWV * WAVE;
    constexpr int EB = NWV * SHAPE;            // experts per block
    constexpr int VN = VecLoad<XT>::N;         // elements per 16 bytes
    constexpr int KC = 16 * VN;                // h per slab: 256 bytes of every token row
    constexpr int XS = KC + 4;                 // padded fp32 row (conflict-free 128-bit row reads)
    constexpr int XPT = RT_TB * 16 / NTH;      // 16-byte x chunks per thread and slab
    constexpr int WQ = KC * EB / (4 * NTH);    // groups of four h of one expert per thread and slab
    // slabs in flight per block: one block holds D x 16 KB of token rows in registers, which is what hides the
    // memory latency when there is only one block of 64 tokens per compute unit
    constexpr int D = NWV == 1 ? 2 : 4;
    constexpr int NACC = SHAPE == 16 ? 16 : 4;
    typedef typename std::conditional<SHAPE == 16, rt_f16, rt_f4>::type acc_t;
    static_assert((KC * EB) % (4 * NTH) == 0, "router slab split");
    __shared__ __align__(16) float xs[RT_TB][XS];
    __shared__ __align__(16) float wsT[EB][KC + 4];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t0 = blockIdx.x * RT_TB, eb0 = blockIdx.y * EB;
    const float* wrow = &wsT[wave * SHAPE + lane % SHAPE][0];
    const float* xrow = &xs[lane][0];
    acc_t acc;
#pragma unroll
    for (int v = 0; v < NACC; ++v) acc[v] = 0.f;

    // Slab s covers h in [ks, ks + KC), ks = min(s * KC, H - KC) (0 when H < KC): the last slab of a row whose
    // length is no multiple of KC overlaps its predecessor and is consumed from offset s * KC - ks on; slabs past
    // the end repeat it and are not consumed at all.  So every slab is a full, in-bounds fetch from a block-uniform
    // base plus lane offsets that never change (the clamps below only matter for H < KC, T and E tails).
    const int ks_max = max(H - KC, 0);
    int xoff[XPT], woff[WQ][4];
#pragma unroll
    for (int i = 0; i < XPT; ++i) {
        const int c = tid + i * NTH;
        xoff[i] = min(c / 16, T - 1 - t0) * H + min((c % 16) * VN, H - VN);
    }
#pragma unroll
    for (int i = 0; i < WQ; ++i) {
        const int c = tid + i * NTH;  // expert c % EB, h 4 * (c / EB) .. + 3 of the slab
#pragma unroll
        for (int q = 0; q < 4; ++q) woff[i][q] = min(4 * (c / EB) + q, H - 1) * E + min(eb0 + c % EB, E - 1);
    }
    const XT* xblk = x + (size_t)t0 * H;

    // slabs wait in registers until their turn in LDS
    rt_u4 xr[D][XPT];  // (vector types, not HIP's uint4 struct: the arrays must stay in registers)
    XT wr[D][WQ][4];
#define RT_FETCH(d, k0)                                                                                      \
    do {                                                                                                     \
        const int ks_ = min((k0), ks_max);                                                                   \
        const XT* xb_ = xblk + ks_;                                                                          \
        const XT* wb_ = w + (size_t)ks_ * E;                                                                 \
        _Pragma("unroll") for (int i = 0; i < XPT; ++i) xr[d][i] = *reinterpret_cast<const rt_u4*>(xb_ + xoff[i]); \
        _Pragma("unroll") for (int i = 0; i < WQ; ++i)                                                        \
            _Pragma("unroll") for (int q = 0; q < 4; ++q) wr[d][i][q] = wb_[woff[i][q]];                      \
    } while (0)
    // registers -> LDS: token rows as fp32 (converted here, once per block, and not by every wave in its MFMA chain),
    // the router slab as fp32, transposed (one 128-bit write per four h)
#define RT_STASH(d)                                                                                                  \
    do {                                                                                                             \
        _Pragma("unroll") for (int i = 0; i < XPT; ++i) {                                                             \
            const int c = tid + i * NTH;                                                                             \
            if constexpr (VN == 8) {                                                                                 \
                const rt_u4 r_ = xr[d][i];                                                                           \
                const rt_f4 lo_ = {__uint_as_float(r_.x << 16), __uint_as_float(r_.x & 0xffff0000u),                 \
                                   __uint_as_float(r_.y << 16), __uint_as_float(r_.y & 0xffff0000u)};                \
                const rt_f4 hi_ = {__uint_as_float(r_.z << 16), __uint_as_float(r_.z & 0xffff0000u),                 \
                                   __uint_as_float(r_.w << 16), __uint_as_float(r_.w & 0xffff0000u)};                \
                *reinterpret_cast<rt_f4*>(&xs[c / 16][(c % 16) * VN]) = lo_;                                         \
                *reinterpret_cast<rt_f4*>(&xs[c / 16][(c % 16) * VN + 4]) = hi_;                                     \
            } else {                                                                                                 \
                *reinterpret_cast<rt_u4*>(&xs[c / 16][(c % 16) * VN]) = xr[d][i];                                    \
            }                                                                                                        \
        }                                                                                                            \
        _Pragma("unroll") for (int i = 0; i < WQ; ++i) {                                                              \
            const int c = tid + i * NTH;                                                                             \
            const rt_f4 v = {load_f32<XT>(&wr[d][i][0]), load_f32<XT>(&wr[d][i][1]), load_f32<XT>(&wr[d][i][2]),     \
                             load_f32<XT>(&wr[d][i][3])};                                                            \
            *reinterpret_cast<rt_f4*>(&wsT[c % EB][4 * (c / EB)]) = v;                                               \
        }                                                                                                            \
    } while (0)

    // One chunk = VN consecutive h of the lane's token row: VN chained MFMAs.  Within one wave a vector
    // instruction does not overlap the chain (measured: one VALU between two dependent MFMAs adds 12 to 14 cycles,
    // a second one 8 more), so the chain's wave does no arithmetic of its own: the operands of the next chunk come
    // out of LDS ready made (token values converted at the stash), read as one group ahead of the chunk's MFMAs.
#define RT_MFMA(XV, WV, u)                                                                                           \
    do {                                                                                                             \
        if constexpr (SHAPE == 16)                                                                                   \
            acc = __builtin_amdgcn_mfma_f32_16x16x1f32(XV[(u) / 4][(u) % 4], WV[(u) / 4][(u) % 4], acc, 0, 0, 0);    \
        else acc = __builtin_amdgcn_mfma_f32_4x4x1f32(XV[(u) / 4][(u) % 4], WV[(u) / 4][(u) % 4], acc, 0, 0, 0);     \
        __builtin_amdgcn_sched_barrier(0);                                                                           \
    } while (0)
    // chunk c: MFMAs on XV / WV, behind the LDS reads of chunk c+1 (at slab offset nxt) into XN / WN
#define RT_CHUNK(XV, WV, XN, WN, nxt)                                                                                \
    do {                                                                                                             \
        _Pragma("unroll") for (int q_ = 0; q_ < VN / 4; ++q_) {                                                       \
            XN[q_] = *reinterpret_cast<const rt_f4*>(xrow + (nxt) + 4 * q_);                                         \
            WN[q_] = *reinterpret_cast<const rt_f4*>(wrow + (nxt) + 4 * q_);                                         \
        }                                                                                                            \
        __builtin_amdgcn_sched_barrier(0);                                                                           \
        RT_MFMA(XV, WV, 0); RT_MFMA(XV, WV, 1); RT_MFMA(XV, WV, 2); RT_MFMA(XV, WV, 3);                              \
        if constexpr (VN == 8) { RT_MFMA(XV, WV, 4); RT_MFMA(XV, WV, 5); RT_MFMA(XV, WV, 6); RT_MFMA(XV, WV, 7); }   \
    } while (0)

    // Every slab slot is fetched and stashed unconditionally (no branch around a load: the compiler then knows how
    // many younger loads are in flight at each stash and waits only for the slab it needs).  The fences keep the
    // first loads in slab order: the scheduler would otherwise issue them last slab first.
#pragma unroll
    for (int d = 0; d < D; ++d) {
        RT_FETCH(d, d * KC);
        __builtin_amdgcn_sched_barrier(0);
    }
    for (int kb = 0; kb < H; kb += D * KC) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int k0 = kb + d * KC;
            RT_STASH(d);
            __syncthreads();
            RT_FETCH(d, k0 + D * KC);
            // only the h that exist take part: a padded step would add +0 and could turn a -0 chain into +0
            const int sh = k0 - min(k0, ks_max);        // where h = k0 sits in the slab
            const int kend = sh + max(min(KC, H - k0), 0);
            if (sh < kend) {
                rt_f4 xa[2], xb[2], wa[2], wb[2];
#pragma unroll
                for (int q = 0; q < VN / 4; ++q) {
                    xa[q] = *reinterpret_cast<const rt_f4*>(xrow + sh + 4 * q);
                    wa[q] = *reinterpret_cast<const rt_f4*>(wrow + sh + 4 * q);
                }
                if (sh == 0 && kend == KC) {
                    // a whole slab: sixteen chunks of straight-line code (the read past the last chunk repeats it)
#define RT_PAIR(c) /* chunks c (even) and c + 1 */                                         \
    RT_CHUNK(xa, wa, xb, wb, ((c) + 1) * VN);                                              \
    RT_CHUNK(xb, wb, xa, wa, ((c) + 2 < 16 ? (c) + 2 : 15) * VN)
                    RT_PAIR(0); RT_PAIR(2); RT_PAIR(4); RT_PAIR(6); RT_PAIR(8); RT_PAIR(10); RT_PAIR(12); RT_PAIR(14);
#undef RT_PAIR
                } else {
                    for (int kk = sh; kk < kend; kk += 2 * VN) {
                        // the chunk past the last one is read from a clamped (valid) place and never used
                        RT_CHUNK(xa, wa, xb, wb, min(kk + VN, KC - VN));
                        if (kk + VN < kend) RT_CHUNK(xb, wb, xa, wa, min(kk + 2 * VN, KC - VN));
                    }
                }
            }
            __syncthreads();
        }
    }
#undef RT_CHUNK
#undef RT_MFMA
#undef RT_STASH
#undef RT_FETCH
    const int e = eb0 + wave * SHAPE + lane % SHAPE;
    if (e < E) {
        const float bv = bias ? bias[e] : 0.f;
#pragma unroll
        for (int v = 0; v < NACC; ++v) {
            const int t = t0 + (SHAPE == 16 ? 16 * (v / 4) + 4 * (lane / 16) + v % 4 : 4 * (lane / 4) + v);
            if (t < T) logits[(size_t)t * E + e] = bias ? __fadd_rn(acc[v], bv) : acc[v];
        }
    }
}

// Softmax gates + top-k.  G lanes cooperate on one token (G = 8,16,32,64); lane gl holds experts
// gl, gl+G, gl+2G, ...  Selection key: (logit descending, expert id ascending).
constexpr int TK_MAXV = 8;  // values per lane -> E <= 8*G

template <int G>
__global__ __launch_bounds__(256) void topk_gate_kernel(const float* __restrict__ logits, int32_t* __restrict__ idx,
                                                         float* __restrict__ gate, int T, int E, int k) {
    constexpr int TPW = WAVE / G;  // tokens per wave
    const int lane = lane_id();
    const int gl = lane % G;
    const int wave_global = (blockIdx.x * blockDim.x + threadIdx.x) / WAVE;
    const int n_waves = (gridDim.x * blockDim.x) / WAVE;
    const float NEG_INF = -__builtin_huge_valf();

    for (int tbase = wave_global * TPW; tbase < T; tbase += n_waves * TPW) {
        const int t = tbase + lane / G;
        const bool live = t < T;
        float v[TK_MAXV];
#pragma unroll
        for (int i = 0; i < TK_MAXV; ++i) {
            const int e = gl + i * G;
            v[i] = (live && e < E) ? logits[(size_t)t * E + e] : NEG_INF;
        }
        unsigned taken = 0;
        float row_max = 0.f;
        float sel_v[MOE_MAX_TOPK];
        int sel_e[MOE_MAX_TOPK];
#pragma unroll
        for (int j = 0; j < MOE_MAX_TOPK; ++j) {
            if (j < k) {
                float bv = NEG_INF;
                int be = 0x7fffffff;
#pragma unroll
                for (int i = 0; i < TK_MAXV; ++i) {
                    const int e = gl + i * G;
                    const bool ok = (e < E) && !((taken >> i) & 1u);
                    // ascending e within the lane: strict > keeps the lower id on ties
                    if (ok && (be == 0x7fffffff || v[i] > bv)) { bv = v[i]; be = e; }
                }
#pragma unroll
                for (int off = G / 2; off >= 1; off >>= 1) {
                    const float ov = __shfl_xor(bv, off, WAVE);
                    const int oe = __shfl_xor(be, off, WAVE);
                    if (oe != 0x7fffffff && (be == 0x7fffffff || ov > bv || (ov == bv && oe < be))) { bv = ov; be = oe; }
                }
                if (be != 0x7fffffff && (be % G) == gl) taken |= 1u << (be / G);
                sel_v[j] = bv;
                sel_e[j] = be;
                if (j == 0) row_max = bv;
            }
        }
        // softmax denominator: per-lane ascending partial sum, then xor butterfly
        float part = 0.f;
#pragma unroll
        for (int i = 0; i < TK_MAXV; ++i) {
            const int e = gl + i * G;
            if (e < E) part += expf(v[i] - row_max);
        }
#pragma unroll
        for (int off = G / 2; off >= 1; off >>= 1) part += __shfl_xor(part, off, WAVE);
        if (live && gl == 0) {
#pragma unroll
            for (int j = 0; j < MOE_MAX_TOPK; ++j) {
                if (j < k) {
                    idx[(size_t)t * k + j] = sel_e[j] == 0x7fffffff ? 0 : sel_e[j];
                    gate[(size_t)t * k + j] = expf(sel_v[j] - row_max) / part;
                }
            }
        }
    }
}

template <typename XT, int SHAPE>
void launch_logits_mfma(const XT* x, const XT* w, const float* bias, float* logits, int T, int H, int E, hipStream_t s) {
    const int gx = ceil_div(T, RT_TB), groups = ceil_div(E, SHAPE);
    if (groups == 1) route_logits_mfma_kernel<XT, SHAPE, 1><<<dim3(gx, 1), WAVE, 0, s>>>(x, w, bias, logits, T, H, E);
    else if (groups == 2) route_logits_mfma_kernel<XT, SHAPE, 2><<<dim3(gx, 1), 2 * WAVE, 0, s>>>(x, w, bias, logits, T, H, E);
    else route_logits_mfma_kernel<XT, SHAPE, 4><<<dim3(gx, ceil_div(groups, 4)), 4 * WAVE, 0, s>>>(x, w, bias, logits, T, H, E);
}

template <typename XT>
int launch_logits(const XT* x, const XT* w, const float* bias, float* logits, int T, int H, int E, hipStream_t s) {
    // 16 experts per instruction when that alone gives every SIMD of the chip a wave, else 4 (four times the waves)
    if (E > 8 && ceil_div(T, RT_TB) * ceil_div(E, 16) >= 1024) launch_logits_mfma<XT, 16>(x, w, bias, logits, T, H, E, s);
    else launch_logits_mfma<XT, 4>(x, w, bias, logits, T, H, E, s);
    return moe_check_launch("route_logits");
}

}  // namespace

extern "C" int moe_route_topk(const void* x, const void* router, const float* bias, int dtype, int T, int H, int E,
                              int k, float* logits_ws, int32_t* topk_idx, float* topk_gate, moe_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    MOE_REQUIRE(T >= 0 && H > 0 && E > 0, MOE_ERR_INVALID, "route_topk: bad shape T=%d H=%d E=%d", T, H, E);
    MOE_REQUIRE(k >= 1 && k <= E, MOE_ERR_INVALID, "route_topk: topk=%d must be in [1, E=%d]", k, E);
    MOE_REQUIRE(k <= MOE_MAX_TOPK, MOE_ERR_UNSUPPORTED, "route_topk: topk=%d > %d", k, MOE_MAX_TOPK);
    MOE_REQUIRE(E <= MOE_MAX_EXPERTS, MOE_ERR_UNSUPPORTED, "route_topk: E=%d > %d", E, MOE_MAX_EXPERTS);
    MOE_REQUIRE(dtype == MOE_F32 || dtype == MOE_BF16, MOE_ERR_INVALID, "route_topk: dtype %d", dtype);
    MOE_REQUIRE((H * dtype_size(dtype)) % 16 == 0, MOE_ERR_INVALID, "route_topk: rows must be 16-byte multiples (H=%d)", H);
    if (T == 0) return MOE_OK;
    MOE_REQUIRE(x && router && logits_ws && topk_idx && topk_gate, MOE_ERR_INVALID, "route_topk: null pointer");
    int rc = dtype == MOE_F32
                 ? launch_logits<float>((const float*)x, (const float*)router, bias, logits_ws, T, H, E, s)
                 : launch_logits<bf16_t>((const bf16_t*)x, (const bf16_t*)router, bias, logits_ws, T, H, E, s);
    if (rc) return rc;
    // lanes per token: the fewest that hold all experts at TK_MAXV per lane (more tokens per wave, fewer shuffles)
    int G = 8;
    while (G < 64 && TK_MAXV * G < E) G *= 2;
    if (E > 8 * G) return moe_fail(MOE_ERR_UNSUPPORTED, "route_topk: E=%d too large", E);
    const int tpw = WAVE / G;
    const int waves = ceil_div(T, tpw);
    const int blocks = min(ceil_div(waves, 4), 4096);
    switch (G) {
        case 8: topk_gate_kernel<8><<<blocks, 256, 0, s>>>(logits_ws, topk_idx, topk_gate, T, E, k); break;
        case 16: topk_gate_kernel<16><<<blocks, 256, 0, s>>>(logits_ws, topk_idx, topk_gate, T, E, k); break;
        case 32: topk_gate_kernel<32><<<blocks, 256, 0, s>>>(logits_ws, topk_idx, topk_gate, T, E, k); break;
        default: topk_gate_kernel<64><<<blocks, 256, 0, s>>>(logits_ws, topk_idx, topk_gate, T, E, k); break;
    }
    return moe_check_launch("topk_gate");
}
