// Per-destination counting, offsets, deterministic payload order, and the row-movement kernels
// (pack into [W,M,H], unpack to [E_l,W,CAP,H] / expert-major [S,H], return pack, combine).
//
// Replaces the Python bucket loop of route_and_pack_padding_free (reference utils.py:204-246),
// build_expert_offsets (utils.py:20-31), _build_dst_offsets (benchmark.py:44-49),
// reorder_flat_to_token_buf (baseline.py:178-222) and the intended token_shuffle kernel
// (layers/token_shuffle.py:31-56; kernels.py:179-205).
//
// Order of rows inside a (dst, el) bucket is ascending token index (utils.py:210-219).  An
// atomic-counter scatter would not reproduce that, so the position of every routed slot is
// computed as   expert_start[ex] + (rows of ex in earlier 64-token blocks) + (rows of ex in
// earlier lanes of this block),  with LDS histograms, a wave prefix scan and per-expert lane masks.
// All integer work: results are bit-exact by construction.
#include "common.h"
#include <atomic>

namespace {

constexpr int CB = MOE_COUNT_BLOCK;  // 64 tokens = one wave per counting block

// ---- 1. per-block histogram: hist[e][b] = #slots of block b routed to expert e --------------------
__global__ __launch_bounds__(256) void block_hist_kernel(const int32_t* __restrict__ idx, int32_t* __restrict__ hist,
                                                          int T, int k, int E, int NB) {
    extern __shared__ int32_t lds_hist[];  // [4][E]
    const int wave = threadIdx.x / WAVE;
    int32_t* my = lds_hist + wave * E;
    for (int i = threadIdx.x; i < 4 * E; i += blockDim.x) lds_hist[i] = 0;
    __syncthreads();
    const int b = blockIdx.x * 4 + wave;
    const int t = b * CB + lane_id();
    if (b < NB && t < T) {
        for (int j = 0; j < k; ++j) {
            const int e = idx[(size_t)t * k + j];
            if ((unsigned)e < (unsigned)E) atomicAdd(&my[e], 1);
        }
    }
    __syncthreads();
    if (b < NB)
        for (int e = lane_id(); e < E; e += WAVE) hist[(size_t)e * NB + b] = my[e];
}

__device__ __forceinline__ int wave_incl_scan(int v) {
#pragma unroll
    for (int off = 1; off < WAVE; off <<= 1) {
        const int o = __shfl_up(v, off, WAVE);
        if (lane_id() >= off) v += o;
    }
    return v;
}

// ---- 2. per-expert exclusive scan over blocks (one wave per expert) --------------------------------
__global__ __launch_bounds__(WAVE) void scan_blocks_kernel(const int32_t* __restrict__ hist, int32_t* __restrict__ base,
                                                            int32_t* __restrict__ counts, int NB) {
    const int e = blockIdx.x;
    int running = 0;
    for (int c = 0; c < NB; c += WAVE) {
        const int b = c + lane_id();
        const int v = b < NB ? hist[(size_t)e * NB + b] : 0;
        const int inc = wave_incl_scan(v);
        if (b < NB) base[(size_t)e * NB + b] = running + inc - v;
        running += __shfl(inc, WAVE - 1, WAVE);
    }
    if (lane_id() == 0) counts[e] = running;
}

// ---- 3. expert prefix -> all count/offset outputs (one wave) ---------------------------------------
// ONE_WAVE = false: every wave of the calling block runs this with the same inputs and writes the same values (es is
// shared; the barrier inside is a block barrier that all of them reach).  ONE_WAVE = true: a single wave runs it, whatever
// else the block holds, and the hand-over through es is a wave-local one (no block barrier in divergent control flow).
template <bool ONE_WAVE>
__device__ __forceinline__ void offsets_body(const int32_t* counts, int E, int W, int32_t* es /*[E+1], LDS*/,
                                             int32_t* expert_start /*[E+1]*/, int32_t* __restrict__ send_counts,
                                             int32_t* __restrict__ expert_offs, int32_t* __restrict__ dst_sizes,
                                             int32_t* __restrict__ dst_offsets, int32_t* __restrict__ caps) {
    const int lane = lane_id();
    const int per = (E + WAVE - 1) / WAVE;
    const int lo = min(lane * per, E), hi = min(lo + per, E);
    int sum = 0, cmax = 0;
    for (int e = lo; e < hi; ++e) { const int c = counts[e]; sum += c; cmax = max(cmax, c); }
    const int incl = wave_incl_scan(sum);
    int run = incl - sum;
    for (int e = lo; e < hi; ++e) { es[e] = run; run += counts[e]; }
    if (lane == WAVE - 1) es[E] = incl;
#pragma unroll
    for (int off = WAVE / 2; off >= 1; off >>= 1) cmax = max(cmax, __shfl_xor(cmax, off, WAVE));
    if constexpr (ONE_WAVE) {
        // the lanes' LDS writes above are read by other lanes of the same wave below
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    } else {
        __syncthreads();
    }
    const int E_l = E / W;
    for (int e = lane; e <= E; e += WAVE) expert_start[e] = es[e];
    for (int e = lane; e < E; e += WAVE) {
        send_counts[e] = counts[e];
        expert_offs[e] = es[e] - es[(e / E_l) * E_l];
    }
    int mmax = 0;
    for (int d = lane; d < W; d += WAVE) {
        const int sz = es[(d + 1) * E_l] - es[d * E_l];
        dst_sizes[d] = sz;
        dst_offsets[d] = es[d * E_l];
        mmax = max(mmax, sz);
    }
#pragma unroll
    for (int off = WAVE / 2; off >= 1; off >>= 1) mmax = max(mmax, __shfl_xor(mmax, off, WAVE));
    if (lane == 0) { caps[0] = max(mmax, 1); caps[1] = max(cmax, 1); }
}

__global__ __launch_bounds__(WAVE) void offsets_kernel(const int32_t* __restrict__ counts, int E, int W,
                                                        int32_t* __restrict__ expert_start /*[E+1]*/,
                                                        int32_t* __restrict__ send_counts, int32_t* __restrict__ expert_offs,
                                                        int32_t* __restrict__ dst_sizes, int32_t* __restrict__ dst_offsets,
                                                        int32_t* __restrict__ caps) {
    __shared__ int32_t es[MOE_MAX_EXPERTS + 1];
    offsets_body<true>(counts, E, W, es, expert_start, send_counts, expert_offs, dst_sizes, dst_offsets, caps);
}

// Steps 2 and 3 in one launch when the histogram is small enough for one workgroup (every wave scans the experts
// w, w + 16, ...; then one wave derives the offsets): a launch saved on a stage that is all launches.
constexpr int SCAN1_MAXCELLS = 1 << 16;
__global__ __launch_bounds__(1024) void scan_offsets_kernel(const int32_t* __restrict__ hist, int32_t* __restrict__ base,
                                                             int32_t* __restrict__ counts, int NB, int E, int W,
                                                             int32_t* __restrict__ expert_start, int32_t* __restrict__ send_counts,
                                                             int32_t* __restrict__ expert_offs, int32_t* __restrict__ dst_sizes,
                                                             int32_t* __restrict__ dst_offsets, int32_t* __restrict__ caps) {
    __shared__ int32_t es[MOE_MAX_EXPERTS + 1];
    __shared__ int32_t s_counts[MOE_MAX_EXPERTS];
    const int wave = threadIdx.x / WAVE, nw = blockDim.x / WAVE;
    for (int e = wave; e < E; e += nw) {
        int running = 0;
        for (int c = 0; c < NB; c += WAVE) {
            const int b = c + lane_id();
            const int v = b < NB ? hist[(size_t)e * NB + b] : 0;
            const int inc = wave_incl_scan(v);
            if (b < NB) base[(size_t)e * NB + b] = running + inc - v;
            running += __shfl(inc, WAVE - 1, WAVE);
        }
        if (lane_id() == 0) { counts[e] = running; s_counts[e] = running; }
    }
    __syncthreads();
    if (wave == 0) offsets_body<true>(s_counts, E, W, es, expert_start, send_counts, expert_offs, dst_sizes, dst_offsets, caps);
}

// ---- 4. stable positions: one wave per 64-token block ----------------------------------------------
// One wave ranks the slots of token block b: the rank of a slot among the block's slots of the same expert is the
// number of lower lanes that hold that expert (a token holds an expert at most once), read off a 64-bit lane
// mask per expert that the wave builds in LDS with one atomic OR per slot.  Called by every thread of a block
// (it contains block barriers); waves without a block pass active = false.
__device__ __forceinline__ void rank_block(const int32_t* __restrict__ idx, const int32_t* base, const int32_t* expert_start,
                                           int32_t* __restrict__ pos, int32_t* __restrict__ row_token, int T, int k, int E,
                                           int NB, int b, bool active, unsigned long long* mask /*[E], LDS, per wave*/) {
    const int lane = lane_id();
    const int t = b * CB + lane;
    const bool live = active && t < T;
    int mine[MOE_MAX_TOPK];
#pragma unroll
    for (int j = 0; j < MOE_MAX_TOPK; ++j) mine[j] = (live && j < k) ? idx[(size_t)t * k + j] : -1;
    if (active)
        for (int e = lane; e < E; e += WAVE) mask[e] = 0ull;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < MOE_MAX_TOPK; ++j)
        if ((unsigned)mine[j] < (unsigned)E) atomicOr(&mask[mine[j]], 1ull << lane);
    __syncthreads();
    const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (WAVE - lane));
#pragma unroll
    for (int j = 0; j < MOE_MAX_TOPK; ++j) {
        const int e = mine[j];
        if ((unsigned)e < (unsigned)E) {
            const int p = expert_start[e] + base[(size_t)e * NB + b] + __popcll(mask[e] & lt_mask);
            pos[(size_t)t * k + j] = p;
            row_token[p] = t;
        }
    }
    __syncthreads();  // the masks are reused by the caller's next block
}

__global__ __launch_bounds__(256) void rank_kernel(const int32_t* __restrict__ idx, const int32_t* __restrict__ base,
                                                    const int32_t* __restrict__ expert_start, int32_t* __restrict__ pos,
                                                    int32_t* __restrict__ row_token, int T, int k, int E, int NB) {
    __shared__ unsigned long long masks[4][MOE_MAX_EXPERTS];
    const int wave = threadIdx.x / WAVE;
    const int b = blockIdx.x * 4 + wave;
    rank_block(idx, base, expert_start, pos, row_token, T, k, E, NB, b, b < NB, masks[wave]);
}

// ---- the four steps above in one block, for few tokens (NB <= CS_MAXNB blocks of 64): launch latency is all that
// such a count costs, so one launch instead of four.  Same arithmetic, tables in LDS instead of the workspace.
constexpr int CS_MAXNB = 16;
constexpr int CS_MAXCELLS = 4096;  // E * NB histogram cells held in LDS (twice: counts and prefixes)

__global__ __launch_bounds__(256) void count_small_kernel(const int32_t* __restrict__ idx, int T, int k, int E, int W, int NB,
                                                           int32_t* __restrict__ send_counts, int32_t* __restrict__ expert_offs,
                                                           int32_t* __restrict__ dst_sizes, int32_t* __restrict__ dst_offsets,
                                                           int32_t* __restrict__ caps, int32_t* __restrict__ pos,
                                                           int32_t* __restrict__ row_token) {
    __shared__ int32_t hist[CS_MAXCELLS];   // [e][b]
    __shared__ int32_t base[CS_MAXCELLS];   // [e][b] rows of e in earlier blocks
    __shared__ int32_t counts[MOE_MAX_EXPERTS];
    __shared__ int32_t es[MOE_MAX_EXPERTS + 1];
    __shared__ int32_t expert_start[MOE_MAX_EXPERTS + 1];
    __shared__ unsigned long long masks[4][MOE_MAX_EXPERTS];
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    for (int i = threadIdx.x; i < E * NB; i += blockDim.x) hist[i] = 0;
    __syncthreads();
    for (int b = wave; b < NB; b += 4) {
        const int t = b * CB + lane;
        if (t < T)
            for (int j = 0; j < k; ++j) {
                const int e = idx[(size_t)t * k + j];
                if ((unsigned)e < (unsigned)E) atomicAdd(&hist[e * NB + b], 1);
            }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        int run = 0;
        for (int b = 0; b < NB; ++b) { base[e * NB + b] = run; run += hist[e * NB + b]; }
        counts[e] = run;
    }
    __syncthreads();
    offsets_body<false>(counts, E, W, es, expert_start, send_counts, expert_offs, dst_sizes, dst_offsets, caps);
    __syncthreads();
    for (int b0 = 0; b0 < NB; b0 += 4)  // (uniform trip count: rank_block holds block barriers)
        rank_block(idx, base, expert_start, pos, row_token, T, k, E, NB, b0 + wave, b0 + wave < NB, masks[wave]);
}

// ---- small integer helpers --------------------------------------------------------------------------
__global__ void max_floor1_kernel(const int32_t* __restrict__ v, int n, int32_t* __restrict__ out) {
    __shared__ int32_t red[256];
    int m = 1;
    for (int i = threadIdx.x; i < n; i += blockDim.x) m = max(m, v[i]);
    red[threadIdx.x] = m;
    __syncthreads();
    for (int s = blockDim.x / 2; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) red[threadIdx.x] = max(red[threadIdx.x], red[threadIdx.x + s]);
        __syncthreads();
    }
    if (threadIdx.x == 0) out[0] = red[0];
}

// Tables derived from recv_counts [W,E_l] (one block):
//   src_off[s*E_l+e] = exclusive prefix over e of recv_counts[s,:]   (row inside slot s)
//   row_off[e*W+s]   = exclusive prefix over flattened (e,s) of recv_counts[s,e]  (+ total at [E_l*W])
//   flat_off[s*E_l+e]= exclusive prefix over flattened (s,e)         (row in a padding-free flat payload)
__global__ __launch_bounds__(WAVE) void recv_tables_kernel(const int32_t* __restrict__ rc, int W, int E_l,
                                                            int32_t* __restrict__ src_off, int32_t* __restrict__ row_off,
                                                            int32_t* __restrict__ flat_off, int32_t* __restrict__ pca,
                                                            int32_t* __restrict__ expert_cnt) {
    const int n = W * E_l;
    const int lane = lane_id();
    const int per = (n + WAVE - 1) / WAVE;
    const int lo = min(lane * per, n), hi = min(lo + per, n);
    // (e,s)-major prefix
    int sum = 0;
    for (int i = lo; i < hi; ++i) sum += rc[(i % W) * E_l + (i / W)];
    int incl = wave_incl_scan(sum);
    int run = incl - sum;
    for (int i = lo; i < hi; ++i) { row_off[i] = run; run += rc[(i % W) * E_l + (i / W)]; }
    if (lane == WAVE - 1) row_off[n] = incl;
    // (s,e)-major prefix
    sum = 0;
    for (int i = lo; i < hi; ++i) sum += rc[i];
    incl = wave_incl_scan(sum);
    run = incl - sum;
    for (int i = lo; i < hi; ++i) { flat_off[i] = run; run += rc[i]; }
    if (lane == WAVE - 1) flat_off[n] = incl;
    // per-source prefix over experts, pca transpose, per-expert totals
    for (int s = lane; s < W; s += WAVE) {
        int r = 0;
        for (int e = 0; e < E_l; ++e) { src_off[s * E_l + e] = r; r += rc[s * E_l + e]; }
    }
    for (int i = lane; i < n; i += WAVE) {
        if (pca) pca[i] = rc[(i % W) * E_l + (i / W)];
    }
    if (expert_cnt)
        for (int e = lane; e < E_l; e += WAVE) {
            int c = 0;
            for (int s = 0; s < W; ++s) c += rc[s * E_l + e];
            expert_cnt[e] = c;
        }
}


// expert_offs[d,e] = exclusive prefix over e of counts[d,:]; dst_sizes / dst_offsets over d (one wave)
__global__ __launch_bounds__(WAVE) void expert_offsets_kernel(const int32_t* __restrict__ counts, int W, int E_l,
                                                               int32_t* __restrict__ expert_offs, int32_t* __restrict__ dst_sizes,
                                                               int32_t* __restrict__ dst_offsets) {
    __shared__ int32_t sizes[MOE_MAX_EXPERTS];
    const int lane = lane_id();
    for (int d = lane; d < W; d += WAVE) {
        int r = 0;
        for (int e = 0; e < E_l; ++e) { expert_offs[d * E_l + e] = r; r += counts[d * E_l + e]; }
        sizes[d] = r;
        if (dst_sizes) dst_sizes[d] = r;
    }
    __syncthreads();
    if (dst_offsets && lane == 0) {
        int r = 0;
        for (int d = 0; d < W; ++d) { dst_offsets[d] = r; r += sizes[d]; }
    }
}

// ---- row movement: dst[r,:] = src[source_row(r),:], or zeros when the row has no source ---------------
// One wave per output row, 16 bytes per lane.  The source row is resolved inside the kernel (no map
// buffer, no extra launch); every quantity involved is wave-uniform.
enum {
    SRC_MAP = 0,      // map[r]                                  (padding-free payload)
    SRC_PACK = 1,     // send slot (d,m) -> token                (fixed [W,M,H] pack)
    SRC_UNPACK = 2,   // expert-major row r -> recv row          (recv [W,M,H] -> [S,H])
    SRC_TOKBUF = 3,   // token_buf row (e,s,j) -> recv row       (recv [W,M,H] -> [E_l,W,CAP,H])
    SRC_RETURN = 4,   // return slot (s,m) -> expert-major row   ([S,H] -> [W,M,H])
    SRC_REORDER = 5,  // token_buf row (e,s,j) -> flat row       (flat payload -> [E_l,W,CAP,H])
    SRC_SHUFFLE = 6,  // expert-major row r -> token_buf row     ([E_l,W,CAP,H] -> [S,H])
    SRC_UNSHUFFLE = 7 // token_buf row (e,s,j) -> expert-major row ([S,H] -> [E_l,W,CAP,H]; the shuffle's gradient)
};

struct RowSource {
    int mode;
    const int32_t* map;                                   // SRC_MAP / SRC_PACK: row_token
    const int32_t *dst_sizes, *dst_offsets;               // SRC_PACK
    const int32_t *rc, *src_off, *row_off, *flat_off;     // recv-driven modes
    int W, E_l, M, CAP;
    int32_t* status;
};

// largest i in [0,n) with off[i] <= r (off ascending, off[0] = 0): the whole wave looks at 64 entries
// at a time and counts them with a ballot.  Equal offsets mark empty segments; the last of a run of
// equal offsets is the segment that owns the row.
__device__ __forceinline__ int wave_seg(const int32_t* __restrict__ off, int n, int r) {
    int total = 0;
    for (int base = 0; base < n; base += WAVE) {
        const int i = base + lane_id();
        const bool le = i < n && off[i] <= r;
        total += __popcll(__ballot(le));
    }
    return total - 1;
}

__device__ __forceinline__ int source_row(const RowSource& a, int r) {
    const int n = a.W * a.E_l;
    switch (a.mode) {
        case SRC_MAP: return a.map[r];
        case SRC_PACK: {
            const int d = r / a.M, m = r % a.M;
            const int cnt = a.dst_sizes[d];
            if (m == 0 && cnt > a.M && a.status && lane_id() == 0) *a.status = 1;
            return m < cnt ? a.map[a.dst_offsets[d] + m] : -1;
        }
        case SRC_UNPACK:
        case SRC_SHUFFLE: {
            if (r >= a.row_off[n]) return -1;
            const int seg = wave_seg(a.row_off, n + 1, r);  // seg = e*W + s
            const int e = seg / a.W, s = seg % a.W, j = r - a.row_off[seg];
            if (a.mode == SRC_SHUFFLE) return (e * a.W + s) * a.CAP + j;
            // a row past the pair capacity never reached the slot (the pack dropped it): it reads as zeros
            const int m = a.src_off[s * a.E_l + e] + j;
            if (m >= a.M) {
                if (a.status && lane_id() == 0) *a.status = 1;
                return -1;
            }
            return s * a.M + m;
        }
        case SRC_TOKBUF:
        case SRC_REORDER: {
            const int j = r % a.CAP, s = (r / a.CAP) % a.W, e = r / (a.CAP * a.W);
            const int c = a.rc[s * a.E_l + e];
            if (j == 0 && c > a.CAP && a.status && lane_id() == 0) *a.status = 1;
            if (j >= c) return -1;
            if (a.mode == SRC_REORDER) return a.flat_off[s * a.E_l + e] + j;
            const int m = a.src_off[s * a.E_l + e] + j;  // row inside the sender's slot; past M it was dropped by the pack
            if (m >= a.M) {
                if (a.status && lane_id() == 0) *a.status = 1;
                return -1;
            }
            return s * a.M + m;
        }
        case SRC_UNSHUFFLE: {
            const int j = r % a.CAP, s = (r / a.CAP) % a.W, e = r / (a.CAP * a.W);
            return j < a.rc[s * a.E_l + e] ? a.row_off[e * a.W + s] + j : -1;
        }
        default: {  // SRC_RETURN
            const int s = r / a.M, m = r % a.M;
            const int32_t* so = a.src_off + s * a.E_l;
            const int tot = so[a.E_l - 1] + a.rc[s * a.E_l + a.E_l - 1];
            if (m >= tot) return -1;
            const int e = wave_seg(so, a.E_l, m);
            return a.row_off[e * a.W + s] + (m - so[e]);
        }
    }
}

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <int WPB>
__global__ __launch_bounds__(WPB * WAVE) void gather_rows_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                                  const RowSource a, int n_rows,
                                                                  int row_vec /* 16-byte units per row */) {
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    for (int r = blockIdx.x * WPB + wave; r < n_rows; r += gridDim.x * WPB) {
        const int m = source_row(a, r);
        u32x4* d = dst + (size_t)r * row_vec;
        if (m >= 0) {
            // streaming copy: every byte is touched once, so loads and stores bypass cache retention
            const u32x4* s = src + (size_t)m * row_vec;
            int c = lane;
            for (; c + 7 * WAVE < row_vec; c += 8 * WAVE) {
                u32x4 v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(s + c + u * WAVE);
#pragma unroll
                for (int u = 0; u < 8; ++u) __builtin_nontemporal_store(v[u], d + c + u * WAVE);
            }
            for (; c < row_vec; c += WAVE) __builtin_nontemporal_store(__builtin_nontemporal_load(s + c), d + c);
        } else {
            const u32x4 z = {0u, 0u, 0u, 0u};
            for (int c = lane; c < row_vec; c += WAVE) __builtin_nontemporal_store(z, d + c);
        }
    }
}

// ---- pack, token-major: every token row is read once and stored to its k send slots ------------------
// Units [0, T) of the launch are tokens (one wave each); the units after them are runs of PACK_ZR consecutive send
// slots each, which only get zeros where they are padding (a wave per slot was mostly wave start-up: with skewed
// routing most of the send buffer is padding).  Same bytes in send_buf as the slot-major gather (SRC_PACK), with x
// read once instead of k times.
constexpr int PACK_ZR = 8;
template <int WPB>
__global__ __launch_bounds__(WPB * WAVE) void pack_tokens_kernel(const u32x4* __restrict__ x, u32x4* __restrict__ send,
                                                                  const int32_t* __restrict__ idx, const int32_t* __restrict__ pos,
                                                                  const int32_t* __restrict__ dst_sizes,
                                                                  const int32_t* __restrict__ dst_offsets, int T, int k, int E_l,
                                                                  int W, int M, int row_vec, int32_t* __restrict__ status,
                                                                  const float* __restrict__ gate, float* __restrict__ send_gate) {
    // gate / send_gate (both or neither): the slot's top-k gate travels with its row, send_gate[d,m] = gate[t,kk], zero
    // in the padding slots -- for a destination that applies the gate to the expert's result before sending it back
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int n_slots = W * M;
    const int n_units = T + (n_slots + PACK_ZR - 1) / PACK_ZR;
    for (int r = blockIdx.x * WPB + wave; r < n_units; r += gridDim.x * WPB) {
        if (r >= T) {
            const int s0 = (r - T) * PACK_ZR, s1 = min(s0 + PACK_ZR, n_slots);
            int d = s0 / M, m = s0 % M;
            int cnt = dst_sizes[d];
            const u32x4 z = {0u, 0u, 0u, 0u};
            for (int sl = s0; sl < s1; ++sl) {
                if (m == 0 && cnt > M && status && lane == 0) *status = 1;
                if (m >= cnt) {
                    u32x4* o = send + (size_t)sl * row_vec;
                    // (ordinary stores: measured 4 to 10 % faster here than non-temporal ones, which win for the copies below)
                    for (int c = lane; c < row_vec; c += WAVE) o[c] = z;
                    if (send_gate && lane == 0) send_gate[sl] = 0.f;
                }
                if (++m == M && sl + 1 < s1) { m = 0; cnt = dst_sizes[++d]; }
            }
            continue;
        }
        // destination rows of the token's k slots (-1: beyond the pair capacity, dropped like the gather drops it)
        int drow[MOE_MAX_TOPK];
#pragma unroll
        for (int j = 0; j < MOE_MAX_TOPK; ++j) {
            drow[j] = -1;
            if (j < k) {
                const int d = idx[(size_t)r * k + j] / E_l;
                const bool d_ok = (unsigned)d < (unsigned)W;  // (an expert id outside [0, W E_l): no slot, and no read of its offset)
                const int m = pos[(size_t)r * k + j] - dst_offsets[d_ok ? d : 0];
                if (d_ok && (unsigned)m < (unsigned)M) drow[j] = d * M + m;
                if (send_gate && drow[j] >= 0 && lane == 0) send_gate[drow[j]] = gate[(size_t)r * k + j];
            }
        }
        const u32x4* src = x + (size_t)r * row_vec;
        // eight 16-byte loads in flight per lane (fewer at the end of a row, or when the row is shorter than 8 KB)
        for (int c = lane; c < row_vec; c += 8 * WAVE) {
            u32x4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (c + u * WAVE < row_vec) v[u] = __builtin_nontemporal_load(src + c + u * WAVE);
#pragma unroll
            for (int j = 0; j < MOE_MAX_TOPK; ++j) {
                if (j < k && drow[j] >= 0) {
                    u32x4* o = send + (size_t)drow[j] * row_vec + c;
#pragma unroll
                    for (int u = 0; u < 8; ++u)
                        if (c + u * WAVE < row_vec) __builtin_nontemporal_store(v[u], o + u * WAVE);
                }
            }
        }
    }
}

// ---- combine: out[t,:] = sum_kk gate[t,kk] * ret[slot(t,kk),:] --------------------------------------
template <typename XT>
struct Vec16;
template <>
struct Vec16<bf16_t> {
    static constexpr int N = 8;
    __device__ static void unpack(const uint4& v, float* f) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) { f[2 * i] = __uint_as_float(w[i] << 16); f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
    }
    __device__ static uint4 pack(const float* f) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = (uint32_t)f32_to_bf16(f[2 * i]) | ((uint32_t)f32_to_bf16(f[2 * i + 1]) << 16);
        return make_uint4(w[0], w[1], w[2], w[3]);
    }
};
template <>
struct Vec16<float> {
    static constexpr int N = 4;
    __device__ static void unpack(const uint4& v, float* f) {
        f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y); f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
    }
    __device__ static uint4 pack(const float* f) {
        return make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3]));
    }
};

// KT = compile-time top-k (1,2,4,8) or 0 for a run-time k up to MOE_MAX_TOPK.  All k row reads of a
// 16-byte column are issued before the first is used.
template <typename XT, int KT, int WPB>
__global__ __launch_bounds__(WPB * WAVE) void combine_kernel(const uint4* __restrict__ ret, const int32_t* __restrict__ idx,
                                                              const int32_t* __restrict__ pos, const float* __restrict__ gate,
                                                              const int32_t* __restrict__ dst_offsets, int T, int k_rt, int E_l,
                                                              int W, int M, int row_vec, uint4* __restrict__ out,
                                                              int32_t* __restrict__ status) {
    constexpr int N = Vec16<XT>::N;
    constexpr int KMAX = KT ? KT : MOE_MAX_TOPK;
    const int k = KT ? KT : k_rt;
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    for (int t = blockIdx.x * WPB + wave; t < T; t += gridDim.x * WPB) {
        // a slot whose destination or row lies outside the [W,M] layout was dropped by the pack (pair capacity
        // exceeded) and has no returned row: it is skipped, like the pack skipped it, and the status word is raised
        size_t rows[KMAX];
        float g[KMAX];
        bool have[KMAX];
#pragma unroll
        for (int j = 0; j < KMAX; ++j) {
            have[j] = false;
            if (j < k) {
                const int d = idx[(size_t)t * k + j] / E_l;
                const bool d_ok = (unsigned)d < (unsigned)W;
                const int m = pos[(size_t)t * k + j] - dst_offsets[d_ok ? d : 0];
                have[j] = d_ok && (unsigned)m < (unsigned)M;
                rows[j] = have[j] ? ((size_t)d * M + m) * row_vec : 0;
                g[j] = gate ? gate[(size_t)t * k + j] : 1.f;  // (no gates: the rows arrive weighted, 1 * x is x exactly)
                if (!have[j] && status && lane == 0) *status = 1;
            }
        }
        // U columns per lane and pass, so that sixteen 16-byte row reads are in flight per lane whatever k is
        constexpr int U = KT ? (KT >= 16 ? 1 : 16 / KT) : 1;
        for (int c0 = lane; c0 < row_vec; c0 += U * WAVE) {
            uint4 v[U][KMAX];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int c = c0 + u * WAVE;
#pragma unroll
                for (int j = 0; j < KMAX; ++j)
                    if (j < k && have[j] && c < row_vec) {
                        // every returned row is read once: no cache retention wanted
                        const u32x4 raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(ret + rows[j] + c));
                        v[u][j] = make_uint4(raw.x, raw.y, raw.z, raw.w);
                    }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int c = c0 + u * WAVE;
                if (c >= row_vec) break;
                float acc[N];
#pragma unroll
                for (int i = 0; i < N; ++i) acc[i] = 0.f;
#pragma unroll
                for (int j = 0; j < KMAX; ++j) {
                    if (j < k && have[j]) {
                        float f[N];
                        Vec16<XT>::unpack(v[u][j], f);
#pragma unroll
                        for (int i = 0; i < N; ++i) acc[i] = __fadd_rn(acc[i], __fmul_rn(g[j], f[i]));
                    }
                }
                const uint4 o = Vec16<XT>::pack(acc);
                const u32x4 ov = {o.x, o.y, o.z, o.w};
                // (non-temporal: an ordinary store is 2 to 4 % faster with 8 KB and 14 KB rows and 6 to 11 % slower with 4 KB rows)
                __builtin_nontemporal_store(ov, reinterpret_cast<u32x4*>(out + (size_t)t * row_vec + c));
            }
        }
    }
}

// ---- gradient of the combine: out[t] = sum_kk gate[t,kk] * ret[slot(t,kk)] ------------------------------------------
//   d ret[slot(t,kk)] = gate[t,kk] * d out[t]        (every slot belongs to one (t,kk): a scatter, like the pack)
//   d gate[t,kk]      = < d out[t], ret[slot(t,kk)] > (fp32 sum over the row: per-lane partial sums in column order, then
//                                                     a butterfly over the lanes -- reproducible from call to call)
// Rows [0, T) of the launch are tokens (one wave each); rows [T, T + W*M) are the slots of d ret, which only get zeros when
// they are padding (no (t,kk) maps there) -- as in pack_tokens_kernel.  Dropped slots (outside [W,M]) get no gradient.
template <typename XT, int WPB>
__global__ __launch_bounds__(WPB * WAVE) void combine_backward_kernel(const uint4* __restrict__ dout, const uint4* __restrict__ ret,
                                                                       const int32_t* __restrict__ idx, const int32_t* __restrict__ pos,
                                                                       const float* __restrict__ gate,
                                                                       const int32_t* __restrict__ dst_sizes,
                                                                       const int32_t* __restrict__ dst_offsets, int T, int k, int E_l,
                                                                       int W, int M, int row_vec, uint4* __restrict__ dret,
                                                                       float* __restrict__ dgate) {
    constexpr int N = Vec16<XT>::N;
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int n_rows = T + W * M;
    for (int r = blockIdx.x * WPB + wave; r < n_rows; r += gridDim.x * WPB) {
        if (r >= T) {
            const int d = (r - T) / M, m = (r - T) % M;
            if (m < dst_sizes[d]) continue;
            uint4* o = dret + (size_t)(r - T) * row_vec;
            for (int c = lane; c < row_vec; c += WAVE) o[c] = make_uint4(0, 0, 0, 0);
            continue;
        }
        const uint4* drow = dout + (size_t)r * row_vec;
        for (int j = 0; j < k; ++j) {
            const int d = idx[(size_t)r * k + j] / E_l;
            const bool d_ok = (unsigned)d < (unsigned)W;
            const int m = pos[(size_t)r * k + j] - dst_offsets[d_ok ? d : 0];
            const bool have = d_ok && (unsigned)m < (unsigned)M;
            const float g = gate[(size_t)r * k + j];
            float dot = 0.f;
            if (have) {
                const size_t slot = ((size_t)d * M + m) * row_vec;
                for (int c = lane; c < row_vec; c += WAVE) {
                    float dv[N], rv[N], ov[N];
                    Vec16<XT>::unpack(drow[c], dv);
                    Vec16<XT>::unpack(ret[slot + c], rv);
#pragma unroll
                    for (int i = 0; i < N; ++i) {
                        dot = __fadd_rn(dot, __fmul_rn(dv[i], rv[i]));
                        ov[i] = __fmul_rn(g, dv[i]);
                    }
                    dret[slot + c] = Vec16<XT>::pack(ov);
                }
            }
#pragma unroll
            for (int off = WAVE / 2; off >= 1; off >>= 1) dot = __fadd_rn(dot, __shfl_xor(dot, off, WAVE));
            if (lane == 0) dgate[(size_t)r * k + j] = dot;
        }
    }
}

template <typename XT>
int launch_combine(const void* ret, const int32_t* idx, const int32_t* pos, const float* gate, const int32_t* dst_offsets, int T,
                   int k, int E_l, int W, int M, int row_vec, void* out, int32_t* status, hipStream_t s) {
    const int blocks = min(ceil_div(T, 4), 65535 * 8);
#define MOE_COMBINE(KT) \
    combine_kernel<XT, KT, 4><<<blocks, 4 * WAVE, 0, s>>>((const uint4*)ret, idx, pos, gate, dst_offsets, T, k, E_l, W, M, row_vec, (uint4*)out, status)
    switch (k) {
        case 1: MOE_COMBINE(1); break;
        case 2: MOE_COMBINE(2); break;
        case 4: MOE_COMBINE(4); break;
        case 8: MOE_COMBINE(8); break;
        default: MOE_COMBINE(0); break;
    }
#undef MOE_COMBINE
    return moe_check_launch("combine");
}

int gather_rows(const void* src, void* dst, const RowSource& a, int n_rows, int row_bytes, hipStream_t s) {
    if (n_rows == 0) return MOE_OK;
    const int blocks = min(ceil_div(n_rows, 4), 65535 * 8);
    gather_rows_kernel<4><<<blocks, 4 * WAVE, 0, s>>>((const u32x4*)src, (u32x4*)dst, a, n_rows, row_bytes / 16);
    return moe_check_launch("gather_rows");
}

// Expert-major row r of the receive side -> row of the [W,M,H] buffer that holds it (one thread per row, binary search in
// the (expert, source)-major prefix).  The same index serves the way back: the result row of r returns to the slot its input
// came from.  Rows past the received total map to row 0; rows the pack dropped (position in the sender's slot at or past
// the pair capacity M) map to -1: the GEMMs read row 0 for them and store nothing.
// One launch: every block derives the two prefix tables it needs from recv_counts in LDS (at most
// MOE_MAX_EXPERTS entries: a wave's scan) instead of waiting for a table kernel; block 0 also leaves the per-expert totals.
// M = 0: the receive buffer is a padding-free flat payload instead (source-major, expert-minor blocks, the layout
// reorder_flat_to_token_buf of the reference reads, baseline.py:204-218): the row of (e, s, j) is the exclusive prefix of the
// counts over flattened (s, e) plus j, and no row can have been dropped.
// recv_gate / row_gate (both or neither): the gates that arrived with the rows, [rows of the receive buffer], gathered
// into expert-major order for the GEMM that applies them (0 for rows without a source).
__global__ __launch_bounds__(256) void row_map_from_counts_kernel(const int32_t* __restrict__ rc, int W, int E_l, int M, int n_rows,
                                                                   int32_t* __restrict__ map, int32_t* __restrict__ expert_cnt,
                                                                   const float* __restrict__ recv_gate, float* __restrict__ row_gate) {
    __shared__ int32_t s_row_off[MOE_MAX_EXPERTS + 1];
    __shared__ int32_t s_src_off[MOE_MAX_EXPERTS];
    const int n = W * E_l;
    const bool flat = M == 0;
    if (threadIdx.x < WAVE) {
        const int lane = lane_id();
        const int per = (n + WAVE - 1) / WAVE;
        const int lo = min(lane * per, n), hi = min(lo + per, n);
        int sum = 0;
        for (int i = lo; i < hi; ++i) sum += rc[(i % W) * E_l + (i / W)];
        const int incl = wave_incl_scan(sum);
        int run = incl - sum;
        for (int i = lo; i < hi; ++i) { s_row_off[i] = run; run += rc[(i % W) * E_l + (i / W)]; }
        if (lane == WAVE - 1) s_row_off[n] = incl;
        if (flat) {  // exclusive prefix over flattened (s, e): where the block of (s, e) starts in the flat payload
            int fsum = 0;
            for (int i = lo; i < hi; ++i) fsum += rc[i];
            const int fincl = wave_incl_scan(fsum);
            int frun = fincl - fsum;
            for (int i = lo; i < hi; ++i) { s_src_off[i] = frun; frun += rc[i]; }
        } else {
            for (int sr = lane; sr < W; sr += WAVE) {
                int r = 0;
                for (int e = 0; e < E_l; ++e) { s_src_off[sr * E_l + e] = r; r += rc[sr * E_l + e]; }
            }
        }
        if (blockIdx.x == 0 && expert_cnt)
            for (int e = lane; e < E_l; e += WAVE) {
                int c = 0;
                for (int sr = 0; sr < W; ++sr) c += rc[sr * E_l + e];
                expert_cnt[e] = c;
            }
    }
    __syncthreads();
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= n_rows) return;
    if (r >= s_row_off[n]) {
        map[r] = 0;
        if (row_gate) row_gate[r] = 0.f;
        return;
    }
    int lo = 0, hi = n;  // s_row_off[0] = 0 <= r; the last of a run of equal offsets owns the row
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (s_row_off[mid] <= r) lo = mid; else hi = mid;
    }
    const int e = lo / W, sr = lo % W;
    const int m = s_src_off[sr * E_l + e] + (r - s_row_off[lo]);
    const int row = flat ? m : (m < M ? sr * M + m : -1);
    map[r] = row;
    if (row_gate) row_gate[r] = row >= 0 ? recv_gate[row] : 0.f;
}

// rows [size_s, M) of every slot s of a [W,M,row] buffer <- 0, size_s = sum over e of rc[s,e]; one wave per run of
// PACK_ZR consecutive rows (the slot's size is summed once per run, or twice when the run crosses into the next slot)
__device__ __forceinline__ int slot_size(const int32_t* __restrict__ rc, int s, int E_l, int lane) {
    int size = 0;
    for (int e = lane; e < E_l; e += WAVE) size += rc[s * E_l + e];
#pragma unroll
    for (int off = WAVE / 2; off >= 1; off >>= 1) size += __shfl_xor(size, off, WAVE);
    return size;
}
__global__ __launch_bounds__(256) void zero_padding_rows_kernel(u32x4* __restrict__ buf, const int32_t* __restrict__ rc, int W,
                                                                 int E_l, int M, int row_vecs) {
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int r0 = (blockIdx.x * (blockDim.x / WAVE) + wave) * PACK_ZR, r1 = min(r0 + PACK_ZR, W * M);
    if (r0 >= r1) return;
    int s = r0 / M, m = r0 % M;
    int size = slot_size(rc, s, E_l, lane);
    const u32x4 z = {0u, 0u, 0u, 0u};
    for (int r = r0; r < r1; ++r) {
        if (m >= size) {
            u32x4* row = buf + (size_t)r * row_vecs;
            for (int c = lane; c < row_vecs; c += WAVE) __builtin_nontemporal_store(z, row + c);
        }
        if (++m == M && r + 1 < r1) { m = 0; size = slot_size(rc, ++s, E_l, lane); }
    }
}

// map_ws of the recv-driven entry points: three prefix tables plus room for a transposed copy of the counts
size_t recv_tables_ints(int W, int E_l) { return (size_t)3 * (W * E_l + 1) + (size_t)W * E_l; }

int check_rows(const char* who, int dtype, int H) {
    if (dtype != MOE_F32 && dtype != MOE_BF16) return moe_fail(MOE_ERR_INVALID, "%s: dtype %d", who, dtype);
    if (H <= 0 || (H * dtype_size(dtype)) % 16 != 0)
        return moe_fail(MOE_ERR_INVALID, "%s: rows must be 16-byte multiples (H=%d)", who, H);
    return MOE_OK;
}

}  // namespace

extern "C" size_t moe_count_workspace_bytes(int T, int k, int E) {
    (void)k;
    const size_t NB = (size_t)ceil_div(T > 0 ? T : 1, CB);
    // hist[E][NB] + base[E][NB] + counts[E] + expert_start[E+1]
    return sizeof(int32_t) * (2 * (size_t)E * NB + 2 * (size_t)E + 1);
}

extern "C" int moe_count_and_offsets(const int32_t* topk_idx, int T, int k, int E, int W, int32_t* send_counts,
                                     int32_t* expert_offs, int32_t* dst_sizes, int32_t* dst_offsets, int32_t* caps,
                                     int32_t* pos, int32_t* row_token, void* ws, size_t ws_bytes, moe_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    MOE_REQUIRE(T >= 0 && E > 0 && W > 0, MOE_ERR_INVALID, "count: bad shape T=%d E=%d W=%d", T, E, W);
    MOE_REQUIRE(E % W == 0, MOE_ERR_INVALID, "num_experts_total must be divisible by world_size (E=%d W=%d)", E, W);
    MOE_REQUIRE(k >= 1 && k <= MOE_MAX_TOPK, MOE_ERR_UNSUPPORTED, "count: topk=%d outside [1,%d]", k, MOE_MAX_TOPK);
    MOE_REQUIRE(E <= MOE_MAX_EXPERTS, MOE_ERR_UNSUPPORTED, "count: E=%d > %d", E, MOE_MAX_EXPERTS);
    MOE_REQUIRE(send_counts && expert_offs && dst_sizes && dst_offsets && caps && ws, MOE_ERR_INVALID, "count: null pointer");
    MOE_REQUIRE(T == 0 || (topk_idx && pos && row_token), MOE_ERR_INVALID, "count: null pointer");
    MOE_REQUIRE(ws_bytes >= moe_count_workspace_bytes(T, k, E), MOE_ERR_WORKSPACE, "count: workspace %zu < %zu", ws_bytes,
                moe_count_workspace_bytes(T, k, E));
    const int NB = ceil_div(T > 0 ? T : 1, CB);
    int32_t* hist = (int32_t*)ws;
    int32_t* base = hist + (size_t)E * NB;
    int32_t* counts = base + (size_t)E * NB;
    int32_t* expert_start = counts + E;
    if (T > 0 && NB <= CS_MAXNB && E * NB <= CS_MAXCELLS) {
        count_small_kernel<<<1, 256, 0, s>>>(topk_idx, T, k, E, W, NB, send_counts, expert_offs, dst_sizes, dst_offsets, caps, pos,
                                             row_token);
        return moe_check_launch("count_and_offsets");
    }
    block_hist_kernel<<<ceil_div(NB, 4), 256, 4 * E * sizeof(int32_t), s>>>(topk_idx, hist, T, k, E, NB);
    if ((long long)E * NB <= SCAN1_MAXCELLS) {
        scan_offsets_kernel<<<1, 1024, 0, s>>>(hist, base, counts, NB, E, W, expert_start, send_counts, expert_offs, dst_sizes,
                                               dst_offsets, caps);
    } else {
        scan_blocks_kernel<<<E, WAVE, 0, s>>>(hist, base, counts, NB);
        offsets_kernel<<<1, WAVE, 0, s>>>(counts, E, W, expert_start, send_counts, expert_offs, dst_sizes, dst_offsets, caps);
    }
    if (T > 0) rank_kernel<<<ceil_div(NB, 4), 256, 0, s>>>(topk_idx, base, expert_start, pos, row_token, T, k, E, NB);
    return moe_check_launch("count_and_offsets");
}

// ---- the same entry point for callers that may not allocate: the workspace is a fixed array in the library's own
// device image instead of a caller buffer.  Each GPU holds its own copy of the array at its own address; the address
// is looked up once per device, with that device current, and kept.
static __device__ __align__(256) unsigned char scratch[MOE_COUNT_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
std::atomic<void*> g_scratch_ptr[MAX_DEVICES];

int count_scratch(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return moe_fail(MOE_ERR_LAUNCH, "count_and_offsets_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= MAX_DEVICES) return moe_fail(MOE_ERR_UNSUPPORTED, "count_and_offsets_static: device %d", dev);
    void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            return moe_fail(MOE_ERR_LAUNCH, "count_and_offsets_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // (racing first calls look up the same address)
    }
    *out = ptr;
    return MOE_OK;
}
}  // namespace

extern "C" size_t moe_count_static_scratch_bytes(void) { return MOE_COUNT_SCRATCH_BYTES; }

extern "C" int moe_count_and_offsets_static(const int32_t* topk_idx, int T, int k, int E, int W, int32_t* send_counts,
                                            int32_t* expert_offs, int32_t* dst_sizes, int32_t* dst_offsets, int32_t* caps,
                                            int32_t* pos, int32_t* row_token, moe_stream_t stream) {
    MOE_REQUIRE(T >= 0 && E > 0 && k >= 1, MOE_ERR_INVALID, "count_and_offsets_static: bad shape T=%d E=%d k=%d", T, E, k);
    const size_t need = moe_count_workspace_bytes(T, k, E);
    MOE_REQUIRE(need <= (size_t)MOE_COUNT_SCRATCH_BYTES, MOE_ERR_WORKSPACE,
                "count_and_offsets_static: T=%d tokens with E=%d experts need %zu bytes of scratch, the built-in array holds %zu "
                "(use moe_count_and_offsets with a workspace of your own)", T, E, need, (size_t)MOE_COUNT_SCRATCH_BYTES);
    void* ws = nullptr;
    const int rc = count_scratch(&ws);
    if (rc) return rc;
    // every cell of the workspace that the kernels read is written earlier in the same call (histogram cells by the
    // block that owns them, prefixes by the scan): nothing has to start at zero, stale contents of an earlier call
    // are never read
    return moe_count_and_offsets(topk_idx, T, k, E, W, send_counts, expert_offs, dst_sizes, dst_offsets, caps, pos, row_token, ws,
                                 (size_t)MOE_COUNT_SCRATCH_BYTES, stream);
}

extern "C" int moe_build_expert_offsets(const int32_t* counts, int W, int E_l, int32_t* expert_offs, int32_t* dst_sizes,
                                        int32_t* dst_offsets, moe_stream_t stream) {
    MOE_REQUIRE(W > 0 && E_l > 0 && W <= MOE_MAX_EXPERTS, MOE_ERR_INVALID, "build_expert_offsets: bad shape W=%d E_l=%d", W, E_l);
    MOE_REQUIRE(counts && expert_offs, MOE_ERR_INVALID, "build_expert_offsets: null pointer");
    expert_offsets_kernel<<<1, WAVE, 0, (hipStream_t)stream>>>(counts, W, E_l, expert_offs, dst_sizes, dst_offsets);
    return moe_check_launch("build_expert_offsets");
}

extern "C" int moe_max_floor1(const int32_t* values, int n, int32_t* out, moe_stream_t stream) {
    MOE_REQUIRE(n >= 0 && out && (n == 0 || values), MOE_ERR_INVALID, "max_floor1: bad arguments");
    max_floor1_kernel<<<1, 256, 0, (hipStream_t)stream>>>(values, n, out);
    return moe_check_launch("max_floor1");
}

extern "C" int moe_pack_payload(const void* x, int dtype, int T, int H, const int32_t* row_token, int R, void* payload,
                                moe_stream_t stream) {
    int rc = check_rows("pack_payload", dtype, H);
    if (rc) return rc;
    MOE_REQUIRE(R >= 0 && T >= 0, MOE_ERR_INVALID, "pack_payload: bad shape");
    if (R == 0) return MOE_OK;
    MOE_REQUIRE(x && row_token && payload, MOE_ERR_INVALID, "pack_payload: null pointer");
    RowSource a{};
    a.mode = SRC_MAP;
    a.map = row_token;
    return gather_rows(x, payload, a, R, H * dtype_size(dtype), (hipStream_t)stream);
}

extern "C" int moe_pack(const void* x, int dtype, int T, int H, const int32_t* row_token, const int32_t* dst_sizes,
                        const int32_t* dst_offsets, int W, int M, void* send_buf, int32_t* map_ws, int32_t* status,
                        moe_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    int rc = check_rows("pack", dtype, H);
    if (rc) return rc;
    MOE_REQUIRE(W > 0 && M >= 1 && T >= 0, MOE_ERR_INVALID, "pack: bad shape W=%d M=%d", W, M);
    MOE_REQUIRE((long long)W * M < (1ll << 31), MOE_ERR_UNSUPPORTED, "pack: W*M too large");
    MOE_REQUIRE(send_buf && dst_sizes && dst_offsets, MOE_ERR_INVALID, "pack: null pointer");
    (void)map_ws;
    RowSource a{};
    a.mode = SRC_PACK;
    a.map = row_token;
    a.dst_sizes = dst_sizes;
    a.dst_offsets = dst_offsets;
    a.M = M;
    a.status = status;
    return gather_rows(x, send_buf, a, W * M, H * dtype_size(dtype), s);
}

extern "C" int moe_pack_tokens_gated(const void* x, int dtype, int T, int H, const int32_t* topk_idx, const int32_t* pos,
                                     const float* gate, int k, int E_l, const int32_t* dst_sizes, const int32_t* dst_offsets, int W,
                                     int M, void* send_buf, float* send_gate, int32_t* status, moe_stream_t stream) {
    int rc = check_rows("pack_tokens", dtype, H);
    MOE_REQUIRE((gate == nullptr) == (send_gate == nullptr), MOE_ERR_INVALID, "pack_tokens: gate and send_gate go together");
    if (rc) return rc;
    MOE_REQUIRE(W > 0 && M >= 1 && T >= 0 && E_l > 0, MOE_ERR_INVALID, "pack_tokens: bad shape W=%d M=%d E_l=%d", W, M, E_l);
    MOE_REQUIRE(k >= 1 && k <= MOE_MAX_TOPK, MOE_ERR_UNSUPPORTED, "pack_tokens: topk=%d outside [1,%d]", k, MOE_MAX_TOPK);
    MOE_REQUIRE((long long)W * M + T < (1ll << 31), MOE_ERR_UNSUPPORTED, "pack_tokens: W*M + T too large");
    MOE_REQUIRE(send_buf && dst_sizes && dst_offsets, MOE_ERR_INVALID, "pack_tokens: null pointer");
    MOE_REQUIRE(T == 0 || (x && topk_idx && pos), MOE_ERR_INVALID, "pack_tokens: null pointer");
    const int n_units = T + ceil_div(W * M, PACK_ZR);
    const int blocks = min(ceil_div(n_units, 4), 65535 * 8);
    pack_tokens_kernel<4><<<blocks, 4 * WAVE, 0, (hipStream_t)stream>>>((const u32x4*)x, (u32x4*)send_buf, topk_idx, pos, dst_sizes,
                                                                        dst_offsets, T, k, E_l, W, M,
                                                                        H * dtype_size(dtype) / 16, status, gate, send_gate);
    return moe_check_launch("pack_tokens");
}

extern "C" int moe_pack_tokens(const void* x, int dtype, int T, int H, const int32_t* topk_idx, const int32_t* pos, int k,
                               int E_l, const int32_t* dst_sizes, const int32_t* dst_offsets, int W, int M, void* send_buf,
                               int32_t* status, moe_stream_t stream) {
    return moe_pack_tokens_gated(x, dtype, T, H, topk_idx, pos, nullptr, k, E_l, dst_sizes, dst_offsets, W, M, send_buf, nullptr,
                                 status, stream);
}

static int recv_driven(const char* who, int mode, const void* src, void* dst, int dtype, int H, const int32_t* rc_dev,
                       int W, int E_l, int M, int CAP, int n_out, int32_t* pca, int32_t* expert_cnt, int32_t* map_ws,
                       int32_t* status, hipStream_t s) {
    int rc = check_rows(who, dtype, H);
    if (rc) return rc;
    MOE_REQUIRE(W > 0 && E_l > 0 && W * E_l <= MOE_MAX_EXPERTS, MOE_ERR_INVALID, "%s: bad W=%d E_l=%d", who, W, E_l);
    MOE_REQUIRE(n_out >= 0 && rc_dev && map_ws, MOE_ERR_INVALID, "%s: bad arguments", who);
    int32_t* tables = map_ws;
    const int n = W * E_l;
    int32_t* src_off = tables;
    int32_t* row_off = tables + (n + 1);
    int32_t* flat_off = tables + 2 * (n + 1);
    recv_tables_kernel<<<1, WAVE, 0, s>>>(rc_dev, W, E_l, src_off, row_off, flat_off, pca, expert_cnt);
    if (n_out == 0) return moe_check_launch(who);
    // (an empty flat payload or gradient has no storage: every output row is then padding and the source is never read)
    MOE_REQUIRE(dst && (src || mode == SRC_REORDER || mode == SRC_UNSHUFFLE), MOE_ERR_INVALID, "%s: null pointer", who);
    RowSource a{};
    a.mode = mode;
    a.rc = rc_dev; a.src_off = src_off; a.row_off = row_off; a.flat_off = flat_off;
    a.W = W; a.E_l = E_l; a.M = M; a.CAP = CAP;
    a.status = status;
    return gather_rows(src, dst, a, n_out, H * dtype_size(dtype), s);
}

extern "C" size_t moe_recv_map_ints(int W, int E_l, int n_out) {
    (void)n_out;  // the per-row map of earlier versions is gone: rows are resolved inside the gather kernel
    return recv_tables_ints(W, E_l);
}

extern "C" int moe_unpack_token_buf(const void* recv, int dtype, int W, int M, int H, const int32_t* recv_counts,
                                    int E_l, int CAP, void* token_buf, int32_t* pca, int32_t* map_ws, int32_t* status,
                                    moe_stream_t stream) {
    MOE_REQUIRE(M >= 1 && CAP >= 1, MOE_ERR_INVALID, "unpack_token_buf: M=%d CAP=%d", M, CAP);
    MOE_REQUIRE((long long)E_l * W * CAP < (1ll << 31), MOE_ERR_UNSUPPORTED, "unpack_token_buf: too many rows");
    return recv_driven("unpack_token_buf", SRC_TOKBUF, recv, token_buf, dtype, H, recv_counts, W, E_l, M, CAP, E_l * W * CAP, pca,
                       nullptr, map_ws, status, (hipStream_t)stream);
}

extern "C" int moe_reorder_flat_to_token_buf(const void* flat, int dtype, int R, int H, const int32_t* recv_counts,
                                             int W, int E_l, int CAP, void* token_buf, int32_t* map_ws, int32_t* status,
                                             moe_stream_t stream) {
    (void)R;
    MOE_REQUIRE(CAP >= 1, MOE_ERR_INVALID, "reorder: CAP=%d", CAP);
    MOE_REQUIRE((long long)E_l * W * CAP < (1ll << 31), MOE_ERR_UNSUPPORTED, "reorder: too many rows");
    return recv_driven("reorder_flat_to_token_buf", SRC_REORDER, flat, token_buf, dtype, H, recv_counts, W, E_l, 1, CAP,
                       E_l * W * CAP, nullptr, nullptr, map_ws, status, (hipStream_t)stream);
}

extern "C" int moe_unpack_expert_major(const void* recv, int dtype, int W, int M, int H, const int32_t* recv_counts,
                                       int E_l, void* shuffled, int S_rows, int32_t* expert_cnt, int32_t* map_ws,
                                       moe_stream_t stream) {
    MOE_REQUIRE(M >= 1, MOE_ERR_INVALID, "unpack_expert_major: M=%d", M);
    return recv_driven("unpack_expert_major", SRC_UNPACK, recv, shuffled, dtype, H, recv_counts, W, E_l, M, 1, S_rows, nullptr,
                       expert_cnt, map_ws, nullptr, (hipStream_t)stream);
}

extern "C" int moe_recv_row_map(const int32_t* recv_counts, int W, int E_l, int M, int n_rows, int32_t* row_map,
                                int32_t* expert_cnt, int32_t* map_ws, moe_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    MOE_REQUIRE(W > 0 && E_l > 0 && W * E_l <= MOE_MAX_EXPERTS, MOE_ERR_INVALID, "recv_row_map: bad W=%d E_l=%d", W, E_l);
    MOE_REQUIRE(M >= 1 && n_rows >= 0 && recv_counts, MOE_ERR_INVALID, "recv_row_map: bad arguments");
    (void)map_ws;  // (the tables of earlier versions live in LDS now)
    MOE_REQUIRE(n_rows == 0 || row_map, MOE_ERR_INVALID, "recv_row_map: null pointer");
    // (one launch: every block rebuilds the prefix tables in LDS; at least one block, for the per-expert totals)
    row_map_from_counts_kernel<<<max(ceil_div(n_rows, 256), 1), 256, 0, s>>>(recv_counts, W, E_l, M, n_rows, row_map, expert_cnt,
                                                                             nullptr, nullptr);
    return moe_check_launch("recv_row_map");
}

extern "C" int moe_recv_row_map_gated(const int32_t* recv_counts, int W, int E_l, int M, int n_rows, const float* recv_gate,
                                      int32_t* row_map, float* row_gate, int32_t* expert_cnt, moe_stream_t stream) {
    MOE_REQUIRE(W > 0 && E_l > 0 && W * E_l <= MOE_MAX_EXPERTS, MOE_ERR_INVALID, "recv_row_map_gated: bad W=%d E_l=%d", W, E_l);
    MOE_REQUIRE(M >= 0 && n_rows >= 0 && recv_counts, MOE_ERR_INVALID, "recv_row_map_gated: bad arguments");
    MOE_REQUIRE((recv_gate == nullptr) == (row_gate == nullptr), MOE_ERR_INVALID, "recv_row_map_gated: recv_gate and row_gate go together");
    MOE_REQUIRE(n_rows == 0 || row_map, MOE_ERR_INVALID, "recv_row_map_gated: null pointer");
    row_map_from_counts_kernel<<<max(ceil_div(n_rows, 256), 1), 256, 0, (hipStream_t)stream>>>(recv_counts, W, E_l, M, n_rows, row_map,
                                                                                               expert_cnt, recv_gate, row_gate);
    return moe_check_launch("recv_row_map_gated");
}

extern "C" int moe_recv_row_map_flat(const int32_t* recv_counts, int W, int E_l, int n_rows, int32_t* row_map, int32_t* expert_cnt,
                                     moe_stream_t stream) {
    return moe_recv_row_map_gated(recv_counts, W, E_l, 0, n_rows, nullptr, row_map, nullptr, expert_cnt, stream);
}

extern "C" int moe_zero_padding_rows(void* buf, int dtype, int W, int M, int H, const int32_t* recv_counts, int E_l,
                                     moe_stream_t stream) {
    int rc = check_rows("zero_padding_rows", dtype, H);
    if (rc) return rc;
    MOE_REQUIRE(W > 0 && E_l > 0 && M >= 1 && buf && recv_counts, MOE_ERR_INVALID, "zero_padding_rows: bad arguments");
    MOE_REQUIRE((long long)W * M < (1ll << 31), MOE_ERR_UNSUPPORTED, "zero_padding_rows: too many rows");
    zero_padding_rows_kernel<<<ceil_div(ceil_div(W * M, PACK_ZR), 4), 256, 0, (hipStream_t)stream>>>((u32x4*)buf, recv_counts, W, E_l, M,
                                                                                  H * dtype_size(dtype) / 16);
    return moe_check_launch("zero_padding_rows");
}

// token_buf -> shuffled: pca is [E_l,W]; the tables kernel wants [W,E_l] counts, so transpose first.
__global__ void transpose_counts_kernel(const int32_t* __restrict__ in, int rows, int cols, int32_t* __restrict__ out) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < rows * cols) out[(i % cols) * rows + (i / cols)] = in[i];
}

extern "C" int moe_shuffle(const void* token_buf, int dtype, int E_l, int W, int CAP, int H, const int32_t* pca,
                           void* shuffled, int S_rows, int32_t* expert_cnt, int32_t* map_ws, moe_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    MOE_REQUIRE(W > 0 && E_l > 0 && W * E_l <= MOE_MAX_EXPERTS && CAP >= 1 && S_rows >= 0 && pca && map_ws,
                MOE_ERR_INVALID, "shuffle: bad arguments");
    // recv_counts[s,e] = pca[e,s], kept behind the tables in map_ws
    int32_t* rc_t = map_ws + 3 * (W * E_l + 1);
    transpose_counts_kernel<<<ceil_div(W * E_l, 256), 256, 0, s>>>(pca, E_l, W, rc_t);
    return recv_driven("shuffle", SRC_SHUFFLE, token_buf, shuffled, dtype, H, rc_t, W, E_l, 1, CAP, S_rows, nullptr, expert_cnt,
                       map_ws, nullptr, s);
}

// gradient of moe_shuffle: grad_token_buf[e,s,j,:] = grad_rows[off[e,s] + j,:] for j < pca[e,s], zeros elsewhere
extern "C" int moe_shuffle_backward(const void* grad_rows, int dtype, int E_l, int W, int CAP, int H, const int32_t* pca,
                                    void* grad_token_buf, int32_t* map_ws, moe_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    MOE_REQUIRE(W > 0 && E_l > 0 && W * E_l <= MOE_MAX_EXPERTS && CAP >= 1 && pca && map_ws, MOE_ERR_INVALID,
                "shuffle_backward: bad arguments");
    MOE_REQUIRE((long long)E_l * W * CAP < (1ll << 31), MOE_ERR_UNSUPPORTED, "shuffle_backward: too many rows");
    int32_t* rc_t = map_ws + 3 * (W * E_l + 1);  // recv_counts[s,e] = pca[e,s], kept behind the tables
    transpose_counts_kernel<<<ceil_div(W * E_l, 256), 256, 0, s>>>(pca, E_l, W, rc_t);
    return recv_driven("shuffle_backward", SRC_UNSHUFFLE, grad_rows, grad_token_buf, dtype, H, rc_t, W, E_l, 1, CAP, E_l * W * CAP,
                       nullptr, nullptr, map_ws, nullptr, s);
}

extern "C" int moe_return_pack(const void* y, int dtype, int S_rows, int H, const int32_t* recv_counts, int W, int E_l,
                               int M, void* ret, int32_t* map_ws, moe_stream_t stream) {
    (void)S_rows;
    MOE_REQUIRE(M >= 1, MOE_ERR_INVALID, "return_pack: M=%d", M);
    MOE_REQUIRE((long long)W * M < (1ll << 31), MOE_ERR_UNSUPPORTED, "return_pack: W*M too large");
    return recv_driven("return_pack", SRC_RETURN, y, ret, dtype, H, recv_counts, W, E_l, M, 1, W * M, nullptr, nullptr, map_ws,
                       nullptr, (hipStream_t)stream);
}

extern "C" int moe_combine_backward(const void* d_out, const void* ret, int dtype, int W, int M, int H, const int32_t* topk_idx,
                                    const int32_t* pos, const float* gate, const int32_t* dst_sizes, const int32_t* dst_offsets,
                                    int T, int k, int E_l, void* d_ret, float* d_gate, moe_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    int rc = check_rows("combine_backward", dtype, H);
    if (rc) return rc;
    MOE_REQUIRE(W > 0 && M >= 1 && T >= 0 && E_l > 0, MOE_ERR_INVALID, "combine_backward: bad shape");
    MOE_REQUIRE(k >= 1 && k <= MOE_MAX_TOPK, MOE_ERR_UNSUPPORTED, "combine_backward: topk=%d outside [1,%d]", k, MOE_MAX_TOPK);
    MOE_REQUIRE((long long)W * M + T < (1ll << 31), MOE_ERR_UNSUPPORTED, "combine_backward: W*M + T too large");
    MOE_REQUIRE(d_ret && dst_sizes && dst_offsets, MOE_ERR_INVALID, "combine_backward: null pointer");
    MOE_REQUIRE(T == 0 || (d_out && ret && topk_idx && pos && gate && d_gate), MOE_ERR_INVALID, "combine_backward: null pointer");
    const int n_rows = T + W * M;
    const int blocks = min(ceil_div(n_rows, 4), 65535 * 8);
    const int row_vec = H * dtype_size(dtype) / 16;
    if (dtype == MOE_F32)
        combine_backward_kernel<float, 4><<<blocks, 4 * WAVE, 0, s>>>((const uint4*)d_out, (const uint4*)ret, topk_idx, pos, gate, dst_sizes,
                                                                      dst_offsets, T, k, E_l, W, M, row_vec, (uint4*)d_ret, d_gate);
    else
        combine_backward_kernel<bf16_t, 4><<<blocks, 4 * WAVE, 0, s>>>((const uint4*)d_out, (const uint4*)ret, topk_idx, pos, gate, dst_sizes,
                                                                       dst_offsets, T, k, E_l, W, M, row_vec, (uint4*)d_ret, d_gate);
    return moe_check_launch("combine_backward");
}

extern "C" int moe_combine(const void* ret, int dtype, int W, int M, int H, const int32_t* topk_idx, const int32_t* pos,
                           const float* gate, const int32_t* dst_offsets, int T, int k, int E_l, void* out,
                           int32_t* status, moe_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    int rc = check_rows("combine", dtype, H);
    if (rc) return rc;
    MOE_REQUIRE(W > 0 && M >= 1 && T >= 0 && E_l > 0, MOE_ERR_INVALID, "combine: bad shape");
    MOE_REQUIRE(k >= 1 && k <= MOE_MAX_TOPK, MOE_ERR_UNSUPPORTED, "combine: topk=%d outside [1,%d]", k, MOE_MAX_TOPK);
    if (T == 0) return MOE_OK;
    MOE_REQUIRE(ret && topk_idx && pos && dst_offsets && out, MOE_ERR_INVALID, "combine: null pointer");  // (gate may be NULL)
    const int row_vec = H * dtype_size(dtype) / 16;
    if (dtype == MOE_F32) return launch_combine<float>(ret, topk_idx, pos, gate, dst_offsets, T, k, E_l, W, M, row_vec, out, status, s);
    return launch_combine<bf16_t>(ret, topk_idx, pos, gate, dst_offsets, T, k, E_l, W, M, row_vec, out, status, s);
}
