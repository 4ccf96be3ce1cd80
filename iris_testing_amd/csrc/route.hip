// Router: logits = x @ W_r (+ bias) with a pinned fp32 reduction order, then softmax gates
// and top-k with wavefront-level reductions.
//
// Replaces the device work of `F.softmax(torch.einsum('th,he->te', tokens, router), dim=-1)`
// followed by `torch.topk(..., topk)` in the reference (utils.py:200-202).
//
// Reduction order (what makes the indices reproducible bit-for-bit on a CPU): h is cut into MOE_ROUTE_SEGMENTS = 8
// contiguous segments of L = ceil(H / 8) rounded up to a multiple of 8 elements (the last ones shorter or empty);
//   s_p        = chain over the h of segment p,  chain = fmaf(x[t,h], w[h,e], chain) in ascending h, chain0 = +0.0f
//   logit[t,e] = ((((((s_0 + s_1) + s_2) + s_3) + s_4) + s_5) + s_6) + s_7, then + bias[e]   (fp32 additions, in this order)
// Eight independent chains per (t,e) instead of one: a chain is a sequence of dependent instructions, and its length,
// not the memory system, bounded the kernel while it ran over all of H.  Every chain is one accumulator element of one
// block walked over its segment in ascending order; the eight partial sums meet in the top-k kernel.  The chains run on
// the matrix cores, but only through K = 1 fp32 MFMAs, which perform exactly one fused multiply-add per output element
// and instruction; MFMAs with K > 1 (and all bf16 ones) sum several products in an order that is not specified and are
// not used.
#include "common.h"
#include <type_traits>

namespace {

constexpr int RT_TB = 64;  // tokens per block: one per lane
constexpr int RT_P = MOE_ROUTE_SEGMENTS;

// length of a segment of the reduction (part of the specification of the logits: the CPU checker evaluates the same)
__host__ __device__ inline int route_segment_len(int H) { return ((H + RT_P - 1) / RT_P + 7) & ~7; }

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
// Block = NWV waves on the same TB x 64 tokens; wave i takes G groups of SHAPE experts, [e0 + (i G + g) SHAPE, + SHAPE),
// and runs the TB x G chains of one h side by side (independent accumulators: their MFMAs follow each other without
// waiting, and each operand register read from LDS serves G or TB instructions).  Both operands are converted to fp32
// on their way into LDS (the lane reads four consecutive h of its own token row, and of its expert in the transposed
// router slab, with one 128-bit read each).
typedef float rt_f4 __attribute__((ext_vector_type(4)));
typedef float rt_f16 __attribute__((ext_vector_type(16)));
typedef unsigned int rt_u4 __attribute__((ext_vector_type(4)));

// One segment chain of a team of NWV waves for NTOK tokens and EB experts: the accumulators of the calling wave.
// TEAM1 = false: the team is the whole workgroup (block barriers around every slab).  TEAM1 = true: the team is the calling
// wave alone (NWV = 1), xs / wsT are its private part of the LDS and the hand-overs between its lanes are wave-local ones,
// so that the waves of a workgroup -- one segment each -- run independently.
template <bool TEAM1>
__device__ __forceinline__ void rt_team_sync() {
    if constexpr (TEAM1) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    } else {
        __syncthreads();
    }
}

template <int SHAPE>
struct RtAcc {
    typedef typename std::conditional<SHAPE == 16, rt_f16, rt_f4>::type type;
};

template <typename XT, int SHAPE, int TB, int G, int NWV, int CPR /* 16-byte chunks of a token row per slab */, bool TEAM1, int D>
__device__ __forceinline__ void route_segment_chain(const XT* __restrict__ x, const XT* __restrict__ w, int T, int Hrow, int E, int seg,
                                                    int t0, int eb0, int tid, int wave, float (*xs)[CPR * VecLoad<XT>::N + 4],
                                                    float (*wsT)[CPR * VecLoad<XT>::N + 4],
                                                    typename RtAcc<SHAPE>::type (&acc)[TB][G]) {
    static_assert(SHAPE == 4 || SHAPE == 16, "experts per MFMA");
    constexpr int NTH = NWV * WAVE;
    constexpr int NTOK = TB * RT_TB;           // tokens per block
    constexpr int EB = NWV * G * SHAPE;        // experts per block
    constexpr int VN = VecLoad<XT>::N;         // elements per 16 bytes
    constexpr int KC = CPR * VN;               // h per slab: CPR x 16 bytes of every token row
    constexpr int NCH = CPR;                   // chunks (VN consecutive h) per slab
    constexpr int XPT = NTOK * CPR / NTH;      // 16-byte x chunks per thread and slab
    constexpr int WQ = KC * EB / (4 * NTH);    // groups of four h of one expert per thread and slab
    // D: slabs in flight per team (in registers, until their turn in LDS)
    constexpr int NACC = SHAPE == 16 ? 16 : 4;
    static_assert((KC * EB) % (4 * NTH) == 0 && (NTOK * CPR) % NTH == 0 && (CPR == 4 || CPR == 8 || CPR == 16), "router slab split");
    static_assert(!TEAM1 || NWV == 1, "a team of one wave");
    const int lane = tid & 63;
    // this team's segment of the reduction: h in [h0, h0 + H) of rows that are Hrow long (H = 0: an empty segment)
    const int seg_len = route_segment_len(Hrow);
    const int h0 = min(seg * seg_len, Hrow);
    const int H = min(seg_len, Hrow - h0);
    const float* wrow[G];
    const float* xrow[TB];
#pragma unroll
    for (int g = 0; g < G; ++g) wrow[g] = &wsT[(wave * G + g) * SHAPE + lane % SHAPE][0];
#pragma unroll
    for (int b = 0; b < TB; ++b) xrow[b] = &xs[b * RT_TB + lane][0];
#pragma unroll
    for (int b = 0; b < TB; ++b)
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int v = 0; v < NACC; ++v) acc[b][g][v] = 0.f;

    // Slab s covers h in [ks, ks + KC), ks = min(s * KC, H - KC) (0 when H < KC): the last slab of a row whose
    // length is no multiple of KC overlaps its predecessor and is consumed from offset s * KC - ks on; slabs past
    // the end repeat it and are not consumed at all.  So every slab is a full, in-bounds fetch from a block-uniform
    // base plus lane offsets that never change (the clamps below only matter for H < KC, T and E tails).
    const int ks_max = max(H - KC, 0);
    int xoff[XPT], woff[WQ][4];
#pragma unroll
    for (int i = 0; i < XPT; ++i) {
        const int c = tid + i * NTH;
        xoff[i] = min(c / CPR, T - 1 - t0) * Hrow + max(min((c % CPR) * VN, H - VN), 0);
    }
#pragma unroll
    for (int i = 0; i < WQ; ++i) {
        const int c = tid + i * NTH;  // expert c % EB, h 4 * (c / EB) .. + 3 of the slab
#pragma unroll
        for (int q = 0; q < 4; ++q) woff[i][q] = max(min(4 * (c / EB) + q, H - 1), 0) * E + min(eb0 + c % EB, E - 1);
    }
    // (an empty segment starts at h0 = Hrow: its clamped, never consumed fetches are moved back inside the rows)
    const int hb = H > 0 ? h0 : 0;
    const XT* xblk = x + (size_t)t0 * Hrow + hb;
    w += (size_t)hb * E;

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
                *reinterpret_cast<rt_f4*>(&xs[c / CPR][(c % CPR) * VN]) = lo_;                                       \
                *reinterpret_cast<rt_f4*>(&xs[c / CPR][(c % CPR) * VN + 4]) = hi_;                                   \
            } else {                                                                                                 \
                *reinterpret_cast<rt_u4*>(&xs[c / CPR][(c % CPR) * VN]) = xr[d][i];                                  \
            }                                                                                                        \
        }                                                                                                            \
        _Pragma("unroll") for (int i = 0; i < WQ; ++i) {                                                              \
            const int c = tid + i * NTH;                                                                             \
            const rt_f4 v = {load_f32<XT>(&wr[d][i][0]), load_f32<XT>(&wr[d][i][1]), load_f32<XT>(&wr[d][i][2]),     \
                             load_f32<XT>(&wr[d][i][3])};                                                            \
            *reinterpret_cast<rt_f4*>(&wsT[c % EB][4 * (c / EB)]) = v;                                               \
        }                                                                                                            \
    } while (0)

    // One chunk = VN consecutive h: per h, the TB x G independent MFMAs of the wave's chains.  The operands of the next
    // chunk come out of LDS ready made (token values converted at the stash), read as one group ahead of the chunk's
    // MFMAs; the wave itself does no arithmetic between its MFMAs.
#define RT_MFMA(XV, WV, u)                                                                                           \
    do {                                                                                                             \
        _Pragma("unroll") for (int b_ = 0; b_ < TB; ++b_)                                                             \
            _Pragma("unroll") for (int g_ = 0; g_ < G; ++g_) {                                                        \
                if constexpr (SHAPE == 16)                                                                           \
                    acc[b_][g_] = __builtin_amdgcn_mfma_f32_16x16x1f32(XV[b_][(u) / 4][(u) % 4], WV[g_][(u) / 4][(u) % 4], acc[b_][g_], 0, 0, 0); \
                else                                                                                                 \
                    acc[b_][g_] = __builtin_amdgcn_mfma_f32_4x4x1f32(XV[b_][(u) / 4][(u) % 4], WV[g_][(u) / 4][(u) % 4], acc[b_][g_], 0, 0, 0); \
            }                                                                                                        \
        __builtin_amdgcn_sched_barrier(0);                                                                           \
    } while (0)
    // chunk c: MFMAs on XV / WV, behind the LDS reads of chunk c+1 (at slab offset nxt) into XN / WN
#define RT_CHUNK(XV, WV, XN, WN, nxt)                                                                                \
    do {                                                                                                             \
        _Pragma("unroll") for (int q_ = 0; q_ < VN / 4; ++q_) {                                                       \
            _Pragma("unroll") for (int b_ = 0; b_ < TB; ++b_)                                                         \
                XN[b_][q_] = *reinterpret_cast<const rt_f4*>(xrow[b_] + (nxt) + 4 * q_);                             \
            _Pragma("unroll") for (int g_ = 0; g_ < G; ++g_)                                                          \
                WN[g_][q_] = *reinterpret_cast<const rt_f4*>(wrow[g_] + (nxt) + 4 * q_);                             \
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
            rt_team_sync<TEAM1>();
            RT_FETCH(d, k0 + D * KC);
            // only the h that exist take part: a padded step would add +0 and could turn a -0 chain into +0
            const int sh = k0 - min(k0, ks_max);        // where h = k0 sits in the slab
            const int kend = sh + max(min(KC, H - k0), 0);
            if (sh < kend) {
                rt_f4 xa[TB][2], xb[TB][2], wa[G][2], wb[G][2];
#pragma unroll
                for (int q = 0; q < VN / 4; ++q) {
#pragma unroll
                    for (int b = 0; b < TB; ++b) xa[b][q] = *reinterpret_cast<const rt_f4*>(xrow[b] + sh + 4 * q);
#pragma unroll
                    for (int g = 0; g < G; ++g) wa[g][q] = *reinterpret_cast<const rt_f4*>(wrow[g] + sh + 4 * q);
                }
                if (sh == 0 && kend == KC) {
                    // a whole slab: NCH chunks of straight-line code (the read past the last chunk repeats it)
#define RT_PAIR(c) /* chunks c (even) and c + 1 */                                         \
    RT_CHUNK(xa, wa, xb, wb, ((c) + 1) * VN);                                              \
    RT_CHUNK(xb, wb, xa, wa, ((c) + 2 < NCH ? (c) + 2 : NCH - 1) * VN)
                    RT_PAIR(0); RT_PAIR(2);
                    if constexpr (NCH >= 8) { RT_PAIR(4); RT_PAIR(6); }
                    if constexpr (NCH == 16) { RT_PAIR(8); RT_PAIR(10); RT_PAIR(12); RT_PAIR(14); }
#undef RT_PAIR
                } else {
                    for (int kk = sh; kk < kend; kk += 2 * VN) {
                        // the chunk past the last one is read from a clamped (valid) place and never used
                        RT_CHUNK(xa, wa, xb, wb, min(kk + VN, KC - VN));
                        if (kk + VN < kend) RT_CHUNK(xb, wb, xa, wa, min(kk + 2 * VN, KC - VN));
                    }
                }
            }
            rt_team_sync<TEAM1>();
        }
    }
#undef RT_CHUNK
#undef RT_MFMA
#undef RT_STASH
#undef RT_FETCH
}

// The segment chains as separate workgroups: grid = (segments, token blocks, expert blocks); every block stores its
// partial sums to its plane of the workspace, and a second kernel (topk_gate_kernel) folds the planes.
template <typename XT, int SHAPE, int TB, int G, int NWV, int CPR>
__global__ __launch_bounds__(NWV * WAVE, (NWV == 4 && TB == 2 ? 2 : 1)) void route_logits_mfma_kernel(const XT* __restrict__ x, const XT* __restrict__ w,
                                                                        float* __restrict__ part /*[RT_P][T][E]*/, int T,
                                                                        int Hrow, int E) {
    constexpr int NTOK = TB * RT_TB, EB = NWV * G * SHAPE, KC = CPR * VecLoad<XT>::N, NACC = SHAPE == 16 ? 16 : 4;
    __shared__ __align__(16) float xs[NTOK][KC + 4];
    __shared__ __align__(16) float wsT[EB][KC + 4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // (the segment is the fastest-running block index: the blocks that are resident together then read whole token
    // rows between them, not the same eighth of every row, which would load the memory channels unevenly)
    const int t0 = blockIdx.y * NTOK, eb0 = blockIdx.z * EB;
    const int seg = blockIdx.x;
    typename RtAcc<SHAPE>::type acc[TB][G];
    route_segment_chain<XT, SHAPE, TB, G, NWV, CPR, false, 2>(x, w, T, Hrow, E, seg, t0, eb0, tid, wave, xs, wsT, acc);
    float* out = part + (size_t)seg * T * E;
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int e = eb0 + (wave * G + g) * SHAPE + lane % SHAPE;
        if (e >= E) continue;
#pragma unroll
        for (int b = 0; b < TB; ++b)
#pragma unroll
            for (int v = 0; v < NACC; ++v) {
                const int t = t0 + b * RT_TB + (SHAPE == 16 ? 16 * (v / 4) + 4 * (lane / 16) + v % 4 : 4 * (lane / 4) + v);
                if (t < T) out[(size_t)t * E + e] = acc[b][g][v];
            }
    }
}

// Softmax gates + top-k.  G lanes cooperate on one token (G = 8,16,32,64); lane gl holds the eight consecutive experts
// 8 gl .. 8 gl + 7 (two 16-byte loads per segment plane when the rows are 16-byte multiples).  Selection key: (logit
// descending, expert id ascending).
constexpr int TK_MAXV = 8;  // values per lane -> E <= 8*G

// The value of the lane `off` away in the butterfly of a reduction over 2 off lanes (off a power of two).  Up to 8 it is
// a DPP move (xor 1, xor 2, then the mirror images within 8 and within 16 lanes: by then the two halves are uniform, so
// any lane of the other half will do); beyond that a cross-lane read.
__device__ __forceinline__ unsigned tk_xchg(int off, unsigned x) {
    switch (off) {
        case 1: return (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0xB1, 0xF, 0xF, false);   // quad_perm [1,0,3,2]
        case 2: return (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x4E, 0xF, 0xF, false);   // quad_perm [2,3,0,1]
        case 4: return (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x141, 0xF, 0xF, false);  // row_half_mirror
        case 8: return (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x140, 0xF, 0xF, false);  // row_mirror
        default: return (unsigned)__shfl_xor((int)x, off, WAVE);
    }
}

// One pass of a wave: TPW = 64 / G tokens from tbase on.  part: the segments' partial sums, plane p at part + p * plane,
// token t's row at t_part * E inside a plane (global workspace: t_part = t, plane = T E; a workgroup's own LDS copy:
// t_part = t - first token of the workgroup).
template <int G>
__device__ __forceinline__ void topk_gate_pass(const float* __restrict__ part, size_t plane, int t_part0, const float* __restrict__ bias,
                                               float* __restrict__ logits, int32_t* __restrict__ idx, float* __restrict__ gate, int T,
                                               int E, int k, int tbase) {
    const int lane = lane_id();
    const int gl = lane % G;
    const float NEG_INF = -__builtin_huge_valf();
    {
        const int t = tbase + lane / G;
        const bool live = t < T;
        float v[TK_MAXV];
        const int e0 = gl * TK_MAXV;
        const bool vec = (E & 3) == 0;  // every row of the planes starts at a multiple of 16 bytes (and e0 is a multiple of 8)
#pragma unroll
        for (int h = 0; h < TK_MAXV / 4; ++h) {
            const int eh = e0 + 4 * h;
            float sum[4] = {NEG_INF, NEG_INF, NEG_INF, NEG_INF};
            if (live && eh < E) {
                // the segments' partial sums in segment order, then the bias: this fixes the logit's bits
                const float* pp = part + (size_t)(t - t_part0) * E + eh;
                if (vec) {  // (eh + 3 < E then)
                    float4 sp[RT_P];
#pragma unroll
                    for (int p = 0; p < RT_P; ++p) sp[p] = *reinterpret_cast<const float4*>(pp + (size_t)p * plane);
                    sum[0] = sp[0].x; sum[1] = sp[0].y; sum[2] = sp[0].z; sum[3] = sp[0].w;
#pragma unroll
                    for (int p = 1; p < RT_P; ++p) {
                        sum[0] = __fadd_rn(sum[0], sp[p].x); sum[1] = __fadd_rn(sum[1], sp[p].y);
                        sum[2] = __fadd_rn(sum[2], sp[p].z); sum[3] = __fadd_rn(sum[3], sp[p].w);
                    }
                } else {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        if (eh + c < E) {
                            float a = pp[c];
#pragma unroll
                            for (int p = 1; p < RT_P; ++p) a = __fadd_rn(a, pp[(size_t)p * plane + c]);
                            sum[c] = a;
                        }
                    }
                }
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    if (eh + c < E && bias) sum[c] = __fadd_rn(sum[c], bias[eh + c]);
                if (vec) *reinterpret_cast<float4*>(logits + (size_t)t * E + eh) = make_float4(sum[0], sum[1], sum[2], sum[3]);
                else {
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        if (eh + c < E) logits[(size_t)t * E + eh + c] = sum[c];
                }
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) v[4 * h + c] = (live && eh + c < E) ? sum[c] : NEG_INF;
        }
        // Selection on order-preserving keys: (logit bits mapped to an unsigned that sorts like the float, -0 counted as
        // +0) in the upper word, ~expert in the lower: the 64-bit maximum is the largest logit and, among equals, the
        // lowest expert.  A taken or absent entry has key 0, below every logit (-inf maps to 0x007fffff).
        unsigned kh[TK_MAXV], kl[TK_MAXV];
#pragma unroll
        for (int i = 0; i < TK_MAXV; ++i) {
            const int e = e0 + i;
            const unsigned u = __float_as_uint(v[i] + 0.f);
            const bool there = live && e < E;
            kh[i] = there ? (u ^ (((unsigned)((int)u >> 31)) | 0x80000000u)) : 0u;
            kl[i] = ~(unsigned)e;
        }
        float row_max = 0.f;
        float my_v = 0.f;  // lane gl keeps selection gl (and gl + G, ...) for the gate it computes below
        int my_e = 0;
        float my_v2 = 0.f;
        int my_e2 = 0;
#pragma unroll
        for (int j = 0; j < MOE_MAX_TOPK; ++j) {
            if (j < k) {
                unsigned long long best = 0;
#pragma unroll
                for (int i = 0; i < TK_MAXV; ++i) {
                    const unsigned long long c = ((unsigned long long)kh[i] << 32) | kl[i];
                    best = c > best ? c : best;
                }
#pragma unroll
                for (int off = 1; off < G; off <<= 1) {
                    const unsigned oh = tk_xchg(off, (unsigned)(best >> 32)), ol = tk_xchg(off, (unsigned)best);
                    const unsigned long long o = ((unsigned long long)oh << 32) | ol;
                    best = o > best ? o : best;
                }
                const unsigned bh = (unsigned)(best >> 32);
                const int be = (int)~(unsigned)best;
                // (the owner drops it from its candidates)
#pragma unroll
                for (int i = 0; i < TK_MAXV; ++i)
                    if (be == e0 + i) kh[i] = 0u;
                const float bv = __uint_as_float((bh & 0x80000000u) ? (bh ^ 0x80000000u) : ~bh);
                if (j == 0) row_max = bv;
                if ((j % G) == gl) {
                    if (j < G) { my_v = bv; my_e = be; }
                    else { my_v2 = bv; my_e2 = be; }
                }
            }
        }
        // softmax denominator: per-lane ascending partial sum, then a butterfly over the token's lanes
        float part_sum = 0.f;
#pragma unroll
        for (int i = 0; i < TK_MAXV; ++i) {
            const int e = e0 + i;
            if (e < E) part_sum += expf(v[i] - row_max);
        }
#pragma unroll
        for (int off = 1; off < G; off <<= 1) part_sum += __uint_as_float(tk_xchg(off, __float_as_uint(part_sum)));
        // lane gl writes selection gl (and gl + G when k > G): one exp and one division per lane instead of k in one lane
        if (live && gl < k) {
            idx[(size_t)t * k + gl] = my_e;
            gate[(size_t)t * k + gl] = expf(my_v - row_max) / part_sum;
        }
        if (live && gl + G < k) {
            idx[(size_t)t * k + gl + G] = my_e2;
            gate[(size_t)t * k + gl + G] = expf(my_v2 - row_max) / part_sum;
        }
    }
}

template <int G>
__global__ __launch_bounds__(256) void topk_gate_kernel(const float* __restrict__ part /*[RT_P][T][E]*/,
                                                         const float* __restrict__ bias, float* __restrict__ logits,
                                                         int32_t* __restrict__ idx, float* __restrict__ gate, int T, int E,
                                                         int k) {
    constexpr int TPW = WAVE / G;  // tokens per wave
    const int wave_global = (blockIdx.x * blockDim.x + threadIdx.x) / WAVE;
    const int n_waves = (gridDim.x * blockDim.x) / WAVE;
    for (int tbase = wave_global * TPW; tbase < T; tbase += n_waves * TPW)
        topk_gate_pass<G>(part, (size_t)T * E, 0, bias, logits, idx, gate, T, E, k, tbase);
}

// Logits and top-k in one launch, for up to 16 experts.  A workgroup takes 64 tokens; wave p runs the chains of segment p for
// all experts (G groups of four), on its own slabs in its own part of the LDS, at its own pace (no block barrier inside the
// reduction); the eight waves then leave their partial sums in LDS, meet once, and each folds the sums of eight of the
// tokens in segment order and selects -- the arithmetic of the two-kernel path (route_segment_chain, topk_gate_pass), without
// the partial sums' trip through memory and without the second launch.
template <typename XT, int G, int CPR, int D>
__global__ __launch_bounds__(RT_P * WAVE, 1) void route_fused_kernel(const XT* __restrict__ x, const XT* __restrict__ w,
                                                                      const float* __restrict__ bias, float* __restrict__ logits,
                                                                      int32_t* __restrict__ idx, float* __restrict__ gate, int T,
                                                                      int Hrow, int E, int k) {
    constexpr int KC = CPR * VecLoad<XT>::N, EB = G * 4;
    __shared__ __align__(16) float xs[RT_P][RT_TB][KC + 4];
    __shared__ __align__(16) float wsT[RT_P][EB][KC + 4];
    static_assert(sizeof(float) * RT_P * RT_TB * EB <= sizeof(float) * RT_P * RT_TB * (KC + 4), "the partial sums reuse the token slabs");
    const int lane = threadIdx.x & 63, seg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int t0 = blockIdx.x * RT_TB;
    rt_f4 acc[1][G];
    route_segment_chain<XT, 4, 1, G, 1, CPR, true, D>(x, w, T, Hrow, E, seg, t0, 0, lane, 0, xs[seg], wsT[seg], acc);
    // partial sums: plane seg, row = token of the workgroup, E columns (lane l holds tokens 4 (l / 4) + v, expert 4 g + l % 4)
    float* part = &xs[0][0][0];
    __syncthreads();  // (every wave is done with its slabs)
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int e = g * 4 + lane % 4;
        if (e < E) {
#pragma unroll
            for (int v = 0; v < 4; ++v) part[((size_t)seg * RT_TB + 4 * (lane / 4) + v) * E + e] = acc[0][g][v];
        }
    }
    __syncthreads();
    // eight lanes per token (eight experts each: E <= 16 takes two of them... G lanes hold 8 G' experts): 8 tokens per wave
    constexpr int TG = 8;
    topk_gate_pass<TG>(part, (size_t)RT_TB * E, t0, bias, logits, idx, gate, T, E, k, t0 + seg * (WAVE / TG));
}

// Block shapes.  Many tokens: 128 tokens per block and slabs of 64 h, so that every wave runs two chains per group of
// experts side by side and T / 128 x 8 segments of blocks are resident together (four blocks of this size fit a
// compute unit's LDS); two waves (one group of four experts each) up to 8 experts, four up to 16; beyond that 16
// experts per instruction and four or eight waves (64 or 128 experts per block).  Few tokens: 64 tokens per block
// and one chain per wave, for four times as many waves.
template <typename XT>
int launch_logits(const XT* x, const XT* w, float* part, int T, int H, int E, hipStream_t s) {
    constexpr int CPR = 64 / VecLoad<XT>::N;  // slabs of 64 h
#define RT_LAUNCH(SHAPEv, TBv, Gv, NWVv, CPRv, gz) \
    route_logits_mfma_kernel<XT, SHAPEv, TBv, Gv, NWVv, CPRv><<<dim3(RT_P, ceil_div(T, TBv * RT_TB), gz), NWVv * WAVE, 0, s>>>(x, w, part, T, H, E)
    if (T <= 2048) {
        if (E <= 4) RT_LAUNCH(4, 1, 1, 1, 16, 1);
        else if (E <= 8) RT_LAUNCH(4, 1, 1, 2, 16, 1);
        else if (E <= 64) RT_LAUNCH(4, 1, 1, 4, 16, ceil_div(E, 16));
        else RT_LAUNCH(16, 1, 1, 4, 16, ceil_div(E, 64));
    } else {
        if (E <= 4) RT_LAUNCH(4, 2, 1, 1, CPR, 1);
        else if (E <= 8) RT_LAUNCH(4, 2, 1, 2, CPR, 1);
        else if (E <= 16) RT_LAUNCH(4, 2, 1, 4, CPR, 1);
        else if (E <= 64) {
            // (fp32 tokens: two token blocks per wave do not fit the registers at this shape -- 18 would be spilled)
            if constexpr (sizeof(XT) == 4) RT_LAUNCH(16, 1, 1, 4, CPR, 1);
            else RT_LAUNCH(16, 2, 1, 4, CPR, 1);
        }
        else RT_LAUNCH(16, 2, 1, 8, CPR, ceil_div(E, 128));
    }
#undef RT_LAUNCH
    return moe_check_launch("route_logits");
}

}  // namespace

extern "C" size_t moe_route_workspace_bytes(int T, int E) {
    return sizeof(float) * (size_t)RT_P * (size_t)(T > 0 ? T : 0) * (size_t)(E > 0 ? E : 0);
}

extern "C" int moe_route_topk(const void* x, const void* router, const float* bias, int dtype, int T, int H, int E,
                              int k, float* logits, int32_t* topk_idx, float* topk_gate, void* ws, size_t ws_bytes,
                              moe_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    MOE_REQUIRE(T >= 0 && H > 0 && E > 0, MOE_ERR_INVALID, "route_topk: bad shape T=%d H=%d E=%d", T, H, E);
    MOE_REQUIRE(k >= 1 && k <= E, MOE_ERR_INVALID, "route_topk: topk=%d must be in [1, E=%d]", k, E);
    MOE_REQUIRE(k <= MOE_MAX_TOPK, MOE_ERR_UNSUPPORTED, "route_topk: topk=%d > %d", k, MOE_MAX_TOPK);
    MOE_REQUIRE(E <= MOE_MAX_EXPERTS, MOE_ERR_UNSUPPORTED, "route_topk: E=%d > %d", E, MOE_MAX_EXPERTS);
    MOE_REQUIRE(dtype == MOE_F32 || dtype == MOE_BF16, MOE_ERR_INVALID, "route_topk: dtype %d", dtype);
    MOE_REQUIRE((H * dtype_size(dtype)) % 16 == 0, MOE_ERR_INVALID, "route_topk: rows must be 16-byte multiples (H=%d)", H);
    if (T == 0) return MOE_OK;
    MOE_REQUIRE(x && router && logits && topk_idx && topk_gate && ws, MOE_ERR_INVALID, "route_topk: null pointer");
    MOE_REQUIRE(ws_bytes >= moe_route_workspace_bytes(T, E), MOE_ERR_WORKSPACE, "route_topk: workspace %zu < %zu", ws_bytes,
                moe_route_workspace_bytes(T, E));
    MOE_REQUIRE((((uintptr_t)ws | (uintptr_t)logits) & 15) == 0, MOE_ERR_INVALID, "route_topk: ws and logits must be 16-byte aligned");
    if (E <= 16 && T > 2048) {
        // few experts, many tokens: logits and top-k in one launch, the partial sums never leave the workgroup (the workspace
        // is not used).  With few tokens the launch would be a handful of workgroups, each walking its rows slab after slab
        // (measured: 22 us against 13 for 512 tokens): those keep the two launches, whose first spreads the segments
        // over eight times as many workgroups.
        // (two or four groups of four experts per wave: a wave's 64 lanes move a slab of 32 h of 8 or 16 experts, no less)
        const int blocks = ceil_div(T, RT_TB);
    // (slabs in flight per wave: four of 32 h or three of 64 h with two groups of experts, two with four -- what the registers hold)
#define RT_FUSED(XTv, Gv, CPRv) \
    route_fused_kernel<XTv, Gv, CPRv, (Gv == 2 ? (CPRv * VecLoad<XTv>::N == 32 ? 4 : 2) : 2)><<<blocks, RT_P * WAVE, 0, s>>>((const XTv*)x, (const XTv*)router, bias, logits, topk_idx, topk_gate, T, H, E, k)
        if (dtype == MOE_F32) {
            if (E <= 8) RT_FUSED(float, 2, 8);
            else RT_FUSED(float, 4, 8);
        } else {
            if (E <= 8) RT_FUSED(bf16_t, 2, 8);  // (slabs of 64 h: 128 contiguous bytes of a token row per request)
            else RT_FUSED(bf16_t, 4, 4);
        }
#undef RT_FUSED
        return moe_check_launch("route_fused");
    }
    float* part = (float*)ws;
    int rc = dtype == MOE_F32 ? launch_logits<float>((const float*)x, (const float*)router, part, T, H, E, s)
                              : launch_logits<bf16_t>((const bf16_t*)x, (const bf16_t*)router, part, T, H, E, s);
    if (rc) return rc;
    // lanes per token: the fewest that hold all experts at TK_MAXV per lane (more tokens per wave, fewer shuffles)
    int G = 8;
    while (G < 64 && TK_MAXV * G < E) G *= 2;
    if (E > 8 * G) return moe_fail(MOE_ERR_UNSUPPORTED, "route_topk: E=%d too large", E);
    const int tpw = WAVE / G;
    const int waves = ceil_div(T, tpw);
    const int blocks = min(ceil_div(waves, 4), 4096);
    switch (G) {
        case 8: topk_gate_kernel<8><<<blocks, 256, 0, s>>>(part, bias, logits, topk_idx, topk_gate, T, E, k); break;
        case 16: topk_gate_kernel<16><<<blocks, 256, 0, s>>>(part, bias, logits, topk_idx, topk_gate, T, E, k); break;
        case 32: topk_gate_kernel<32><<<blocks, 256, 0, s>>>(part, bias, logits, topk_idx, topk_gate, T, E, k); break;
        default: topk_gate_kernel<64><<<blocks, 256, 0, s>>>(part, bias, logits, topk_idx, topk_gate, T, E, k); break;
    }
    return moe_check_launch("topk_gate");
}
