// Router: logits = x @ W_r (+ bias) with a pinned fp32 reduction order, then softmax gates
// and top-k with wavefront-level reductions.
//
// Replaces the device work of `F.softmax(torch.einsum('th,he->te', tokens, router), dim=-1)`
// followed by `torch.topk(..., topk)` in the reference (utils.py:200-202).
//
// Reduction order (what makes the indices reproducible bit-for-bit on a CPU):
//   logit[t,e] = bias[e] + chain,  chain = fmaf(x[t,h], w[h,e], chain) for h = 0..H-1, chain0 = +0.0f
// Every (t,e) chain lives in ONE thread; H is walked in ascending order through LDS tiles, so no
// cross-lane or cross-block partial sums exist.  MFMA is deliberately not used here: its internal
// summation order is not specified.
#include "common.h"

namespace {

constexpr int RT_THREADS = 256;
constexpr int RT_KC = 32;  // h per LDS tile
constexpr int RT_TB = 64;  // tokens per block

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

// Block = 256 threads = NEX expert-threads x NTY token-threads; thread computes TT tokens x EE experts.
template <typename XT, int TT, int EE, int NEX>
__global__ __launch_bounds__(RT_THREADS) void route_logits_kernel(const XT* __restrict__ x,
                                                                   const XT* __restrict__ w,
                                                                   const float* __restrict__ bias,
                                                                   float* __restrict__ logits, int T, int H, int E) {
    constexpr int NTY = RT_THREADS / NEX;
    constexpr int TB = NTY * TT;
    constexpr int EB = NEX * EE;
    static_assert(TB == RT_TB, "token tile");
    constexpr int XS = TB + 4;  // padded row stride (keeps 16-byte alignment of the per-thread token vector)
    __shared__ __align__(16) float xs[RT_KC][XS];
    __shared__ __align__(16) float ws[RT_KC][EB];

    const int tid = threadIdx.x;
    const int tx = tid % NEX, ty = tid / NEX;
    const int t0 = blockIdx.x * TB, e0 = blockIdx.y * EB;

    float acc[TT][EE];
#pragma unroll
    for (int i = 0; i < TT; ++i)
#pragma unroll
        for (int j = 0; j < EE; ++j) acc[i][j] = 0.0f;

    constexpr int VN = VecLoad<XT>::N;
    constexpr int CH_PER_TOK = RT_KC / VN;
    constexpr int X_CHUNKS = TB * CH_PER_TOK;
    constexpr int XPT = (X_CHUNKS + RT_THREADS - 1) / RT_THREADS;
    constexpr int WPT = RT_KC * EB / RT_THREADS;
    static_assert(X_CHUNKS % RT_THREADS == 0 && (RT_KC * EB) % RT_THREADS == 0, "staging split");

    // The next slab is fetched into registers (from clamped, always valid addresses) while the current one
    // is consumed; masking and conversion to fp32 happen when it is written to LDS.
    uint4 xr[XPT];
    XT wr[WPT];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < XPT; ++i) {
            const int c = tid + i * RT_THREADS;
            const int tt = c / CH_PER_TOK, kc = (c % CH_PER_TOK) * VN;
            xr[i] = *reinterpret_cast<const uint4*>(x + (size_t)min(t0 + tt, T - 1) * H + min(k0 + kc, H - VN));
        }
#pragma unroll
        for (int i = 0; i < WPT; ++i) {
            const int c = tid + i * RT_THREADS;
            wr[i] = w[(size_t)min(k0 + c / EB, H - 1) * E + min(e0 + c % EB, E - 1)];
        }
    };
    auto stash = [&](int k0) {
#pragma unroll
        for (int i = 0; i < XPT; ++i) {
            const int c = tid + i * RT_THREADS;
            const int tt = c / CH_PER_TOK, kc = (c % CH_PER_TOK) * VN;
            const bool ok = t0 + tt < T && k0 + kc < H;
            float v[VN];
            VecLoad<XT>::unpack(xr[i], v);
#pragma unroll
            for (int j = 0; j < VN; ++j) xs[kc + j][tt] = ok ? v[j] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < WPT; ++i) {
            const int c = tid + i * RT_THREADS;
            const bool ok = k0 + c / EB < H && e0 + c % EB < E;
            ws[c / EB][c % EB] = ok ? load_f32<XT>(&wr[i]) : 0.0f;
        }
    };

    constexpr int UK = 8;  // h per inner step: all LDS reads of the step are issued before its fmaf chains
    fetch(0);
    for (int k0 = 0; k0 < H; k0 += RT_KC) {
        stash(k0);
        __syncthreads();
        if (k0 + RT_KC < H) fetch(k0 + RT_KC);
        const int kmax = min(RT_KC, H - k0);
        int kk = 0;
        for (; kk + UK <= kmax; kk += UK) {
            float xv[UK][TT], wv[UK][EE];
#pragma unroll
            for (int u = 0; u < UK; ++u) {
#pragma unroll
                for (int i = 0; i < TT; ++i) xv[u][i] = xs[kk + u][ty * TT + i];
#pragma unroll
                for (int j = 0; j < EE; ++j) wv[u][j] = ws[kk + u][tx * EE + j];
            }
#pragma unroll
            for (int u = 0; u < UK; ++u)
#pragma unroll
                for (int i = 0; i < TT; ++i)
#pragma unroll
                    for (int j = 0; j < EE; ++j) acc[i][j] = fmaf(xv[u][i], wv[u][j], acc[i][j]);
        }
        for (; kk < kmax; ++kk) {
#pragma unroll
            for (int i = 0; i < TT; ++i)
#pragma unroll
                for (int j = 0; j < EE; ++j) acc[i][j] = fmaf(xs[kk][ty * TT + i], ws[kk][tx * EE + j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < TT; ++i) {
        const int t = t0 + ty * TT + i;
        if (t >= T) continue;
#pragma unroll
        for (int j = 0; j < EE; ++j) {
            const int e = e0 + tx * EE + j;
            if (e < E) logits[(size_t)t * E + e] = bias ? __fadd_rn(acc[i][j], bias[e]) : acc[i][j];
        }
    }
}

// Few experts (E <= 16): one thread per (token, EE experts).  Lane = token (64 tokens per block), wave w
// owns experts [w*EE, w*EE+EE).  x goes through LDS in its storage type (the lane reads its own row 16
// bytes at a time); the router slab is converted to fp32 once per slab and read back with broadcast
// 128-bit LDS reads.  The next slab is fetched into registers while the current one is consumed.
// Same reduction order as above: one fmaf chain per (t,e), ascending h.
constexpr int RS_KC = 128;

template <typename XT, int EE>
__global__ __launch_bounds__(RT_THREADS) void route_logits_small_kernel(const XT* __restrict__ x, const XT* __restrict__ w,
                                                                         const float* __restrict__ bias,
                                                                         float* __restrict__ logits, int T, int H, int E) {
    constexpr int VN = VecLoad<XT>::N;          // elements per 16 bytes
    constexpr int XS = RS_KC + VN;              // padded row (16 bytes of padding: conflict-free b128 rows)
    constexpr int XCH = RT_TB * (RS_KC / VN);   // 16-byte chunks of an x slab
    constexpr int XPT = XCH / RT_THREADS;       // per thread
    constexpr int WPT = 16 * RS_KC / RT_THREADS;  // router elements per thread per slab (16 expert rows)
    __shared__ __align__(16) XT xs[RT_TB][XS];
    __shared__ __align__(16) float wsT[16][RS_KC + 4];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t0 = blockIdx.x * RT_TB;
    const int e0 = wave * EE;
    float acc[EE];
#pragma unroll
    for (int j = 0; j < EE; ++j) acc[j] = 0.f;

    // raw slab data held in registers while the previous slab is consumed; masking and conversion
    // happen when it is written to LDS, so nothing waits on these loads until then
    uint4 xr[XPT];
    XT wr[WPT];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < XPT; ++i) {
            const int c = tid + i * RT_THREADS;
            const int row = c / (RS_KC / VN), col = (c % (RS_KC / VN)) * VN;
            // clamped (always valid) address: no divergent branch, all loads of a slab in flight together
            xr[i] = *reinterpret_cast<const uint4*>(x + (size_t)min(t0 + row, T - 1) * H + min(k0 + col, H - VN));
        }
#pragma unroll
        for (int i = 0; i < WPT; ++i) {
            const int c = tid + i * RT_THREADS;
            wr[i] = w[(size_t)min(k0 + c / 16, H - 1) * E + min(c % 16, E - 1)];
        }
    };
    auto stash = [&](int k0) {
#pragma unroll
        for (int i = 0; i < XPT; ++i) {
            const int c = tid + i * RT_THREADS;
            const int row = c / (RS_KC / VN), col = (c % (RS_KC / VN)) * VN;
            const bool ok = t0 + row < T && k0 + col < H;
            *reinterpret_cast<uint4*>(&xs[row][col]) =
                make_uint4(ok ? xr[i].x : 0u, ok ? xr[i].y : 0u, ok ? xr[i].z : 0u, ok ? xr[i].w : 0u);
        }
#pragma unroll
        for (int i = 0; i < WPT; ++i) {
            const int c = tid + i * RT_THREADS;
            const bool ok = k0 + c / 16 < H && c % 16 < E;
            wsT[c % 16][c / 16] = ok ? load_f32<XT>(&wr[i]) : 0.f;
        }
    };

    constexpr int UN = 4;  // 16-byte x chunks consumed per inner step
    fetch(0);
    for (int k0 = 0; k0 < H; k0 += RS_KC) {
        stash(k0);
        __syncthreads();
        if (k0 + RS_KC < H) fetch(k0 + RS_KC);
        const int kmax = min(RS_KC, H - k0);
        int kk = 0;
        for (; kk + UN * VN <= kmax; kk += UN * VN) {
            // all LDS reads of the step first, then the fmaf chains in ascending h
            uint4 xraw[UN];
            float4 wv[EE][UN * VN / 4];
#pragma unroll
            for (int u = 0; u < UN; ++u) xraw[u] = *reinterpret_cast<const uint4*>(&xs[lane][kk + u * VN]);
#pragma unroll
            for (int j = 0; j < EE; ++j)
#pragma unroll
                for (int q = 0; q < UN * VN / 4; ++q) wv[j][q] = *reinterpret_cast<const float4*>(&wsT[e0 + j][kk + 4 * q]);
#pragma unroll
            for (int u = 0; u < UN; ++u) {
                float xv[VN];
                VecLoad<XT>::unpack(xraw[u], xv);
#pragma unroll
                for (int q = 0; q < VN; q += 4) {
#pragma unroll
                    for (int j = 0; j < EE; ++j) {
                        const float4 wq = wv[j][(u * VN + q) / 4];
                        acc[j] = fmaf(xv[q + 0], wq.x, acc[j]);
                        acc[j] = fmaf(xv[q + 1], wq.y, acc[j]);
                        acc[j] = fmaf(xv[q + 2], wq.z, acc[j]);
                        acc[j] = fmaf(xv[q + 3], wq.w, acc[j]);
                    }
                }
            }
        }
        for (; kk < kmax; kk += VN) {
            float xv[VN];
            VecLoad<XT>::load(&xs[lane][kk], xv);
#pragma unroll
            for (int q = 0; q < VN; q += 4) {
#pragma unroll
                for (int j = 0; j < EE; ++j) {
                    const float4 wq = *reinterpret_cast<const float4*>(&wsT[e0 + j][kk + q]);
                    acc[j] = fmaf(xv[q + 0], wq.x, acc[j]);
                    acc[j] = fmaf(xv[q + 1], wq.y, acc[j]);
                    acc[j] = fmaf(xv[q + 2], wq.z, acc[j]);
                    acc[j] = fmaf(xv[q + 3], wq.w, acc[j]);
                }
            }
        }
        __syncthreads();
    }
    const int t = t0 + lane;
    if (t < T) {
#pragma unroll
        for (int j = 0; j < EE; ++j) {
            const int e = e0 + j;
            if (e < E) logits[(size_t)t * E + e] = bias ? __fadd_rn(acc[j], bias[e]) : acc[j];
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

template <typename XT>
int launch_logits(const XT* x, const XT* w, const float* bias, float* logits, int T, int H, int E, hipStream_t s) {
    const int gx = ceil_div(T, RT_TB);
    if (E <= 4) {
        route_logits_small_kernel<XT, 1><<<gx, RT_THREADS, 0, s>>>(x, w, bias, logits, T, H, E);
    } else if (E <= 8) {
        route_logits_small_kernel<XT, 2><<<gx, RT_THREADS, 0, s>>>(x, w, bias, logits, T, H, E);
    } else if (E <= 12) {
        route_logits_small_kernel<XT, 3><<<gx, RT_THREADS, 0, s>>>(x, w, bias, logits, T, H, E);
    } else if (E <= 16) {
        route_logits_small_kernel<XT, 4><<<gx, RT_THREADS, 0, s>>>(x, w, bias, logits, T, H, E);
    } else if (E <= 32) {
        route_logits_kernel<XT, 2, 4, 8><<<dim3(gx, 1), RT_THREADS, 0, s>>>(x, w, bias, logits, T, H, E);
    } else if (gx * ceil_div(E, 64) < 2 * 256) {
        // too few 64 x 64 blocks to give every SIMD two waves: halve the expert tile instead
        route_logits_kernel<XT, 2, 4, 8><<<dim3(gx, ceil_div(E, 32)), RT_THREADS, 0, s>>>(x, w, bias, logits, T, H, E);
    } else {
        route_logits_kernel<XT, 4, 4, 16><<<dim3(gx, ceil_div(E, 64)), RT_THREADS, 0, s>>>(x, w, bias, logits, T, H, E);
    }
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
    int G = 8;
    while (G < 64 && G < E) G *= 2;
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
