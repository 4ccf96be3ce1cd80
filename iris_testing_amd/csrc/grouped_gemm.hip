// Persistent grouped expert GEMM / MLP on gfx950 MFMA (bf16 and OCP fp8) with LDS-staged tiles,
// plus an fp32 path for the plumbing-size workload.
//
// Replaces the reference's intended expert layer (layers/expert.py:31-60) and grouped_gemm kernel
// (kernels.py:240-289): out[rows of group g] = tokens[rows of g] @ weights[g], fp32 accumulate,
// persistent grid walking a tile list that spans all groups.  Differences in kind, not a port:
//   * tiles are 256 (or 128) x 256, four wave64s each owning a 128 (64) x 128 block of 16x16x32 (bf16) or
//     32x32x64 (fp8) MFMAs with the accumulators in the accumulation registers;
//   * operands go HBM -> LDS directly (global_load_lds, 16 bytes per lane) through a ring of four
//     64-byte K stages; the loads of a stage are spread evenly over one MFMA block and issued more than two
//     blocks ahead; an XOR swizzle of the 16-byte chunks keeps MFMA fragment reads bank-conflict free;
//   * one MFMA block per stage: fragment reads and loads are interleaved one by one between its MFMAs;
//   * weights are re-tiled once into a K-contiguous layout (gate/up interleaved for SwiGLU) so both
//     MFMA operands are read as 128-bit fragments;
//   * ragged group tails are masked (the reference assumes full tiles, kernels.py:270,282);
//   * the tile walk is XCD-aware: the 32 workgroups that share an L2 take a compact 4 x 8 patch of
//     a 16 x 16 super-tile;
//   * a last round of the persistent grid that would leave most compute units idle is split along K over all
//     of them (second launch + a reduction kernel that applies the epilogue), given a workspace.
#include "common.h"
#include <algorithm>
#include <type_traits>

namespace moe_gg {

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int ROWB = 64;   // bytes of K per tile row per LDS ring stage
constexpr int CHUNKS = ROWB / 16;
constexpr int NRING = 4;   // LDS ring stages
constexpr int WROWS = 64 / CHUNKS;  // tile rows moved by one wave-wide 16-byte-per-lane load
constexpr int SUP = 16;  // super-tile edge, in tiles
constexpr int GG_MAXG = MOE_MAX_EXPERTS;
constexpr int GG_BN = 256;
#ifndef GG_BIG_NWM
#define GG_BIG_NWM 2  // waves along M of the 256-row tile (x 2 along N)
#endif
#ifndef GG_FP8_NWM
#define GG_FP8_NWM 4  // fp8: 4 x 2 waves of 64 x 128 each, two per SIMD (measured 3.5 to 7 % faster over the fp8 workloads than 2 x 2
                      // waves of 128 x 128; the same shape costs bf16 5 %)
#endif

#ifndef GG_FP8_BSA_NWM
#define GG_FP8_BSA_NWM 4  // the fp8 down projection (block-scaled activations): waves along M, as for the other fp8 GEMM
#endif

struct GemmParams {
    const uint8_t* A;         // [S_rows, K] activations (bf16 or fp8)
    const uint8_t* B;         // packed weights [E_l, Npad, K]
    void* C;                  // [S_rows, ldc] bf16
    void* C2;                 // optional (bf16 kernels with an activation): the values BEFORE the activation, bf16, row pitch ldc
                              // (SwiGLU: 2 ldc, in the packed gate / up column order), kept for the backward pass
    const int32_t* cnt;       // [E_l] rows per group
    const float* row_scale;   // fp8: [S_rows] per-row activation scale; bf16 with EPI_GATE: [S_rows] per-row gate
    const float* col_scale;   // fp8: [E_l, ncs] per-output-channel scale (gate for SwiGLU)
    const float* col_scale2;  // fp8 SwiGLU: [E_l, ncs] up scales
    // fp8, block-scaled hidden activation (one power-of-two scale, an E8M0 exponent byte, per row and 32 columns; bs_pitch
    // bytes per row): written beside the codes by the gate/up kernel's epilogue (c_bscale, rows as C's), read by the down
    // kernel as the scale operand of its MFMAs (a_bscale, rows as A's).
    uint8_t* c_bscale;
    const uint8_t* a_bscale;
    int bs_pitch;
    const int32_t* a_map;     // optional: logical row -> row of A (gather while loading), else A is row r itself
    const int32_t* c_map;     // optional: logical row -> row of C (scatter while storing)
    int E_l, K, N, Npad, ldc, S_rows, ncs;
    // Optional split of the last, partly filled round of the persistent grid along K: when that round holds at
    // most a quarter of a grid of tiles, each of them is cut into P parts of the K range, one per otherwise idle
    // workgroup, which store their fp32 partial sums here (max_units part tiles of BM x 256 floats); a second
    // kernel adds the parts of a tile in part order and applies the epilogue.  NULL: no split.
    float* part_ws;
    int max_units;
    // Weight-gradient mode (template flag DW): C[g] (dw_rows x N, at C + g * c_group_stride elements) = A_g^T-like product
    // whose reduction runs over the rows of group g.  A is then the TRANSPOSED activation matrix [dw_rows, K] with
    // K = the padded row total (every group's rows padded to a multiple of 64, zero filled), B the output gradients
    // re-tiled like weights over the same padded rows; group g owns K stages [kstart_g, kstart_g + 2 ceil(cnt_g / 64)).
    int dw_rows;
    int dw_src_rows;  // rows of the untransposed operands: the counts are clamped to it, as the operand kernels clamp them
    size_t c_group_stride;
    // Time stamps (the TRACE instantiation only; see moe_diag_gemm_trace): GG_TRACE_TILE_WORDS words per workgroup -- for
    // every tile the wall clock (100 MHz) at the start of its K loop, at the end of its K loop and at the end of its
    // epilogue -- then GG_TRACE_BLOCK_WORDS words of workgroup 0: the clock at the end of each of its MFMA blocks.
    // trace_flags & 1: the epilogue computes but stores nothing.
    unsigned long long* trace;
    int trace_flags;
};
constexpr int GG_TRACE_TILE_WORDS = 256, GG_TRACE_BLOCK_WORDS = 4096;

constexpr int GG_MAX_PARTS = 16;   // parts per tile at most
constexpr int GG_RED_SLABS = 32;   // blocks per tile in the reduction of the parts
constexpr int GG_MIN_PART_STAGES = 8;  // K stages per part at least (64 bytes of K each)

// stages per part when nk stages (even) are cut into P parts: even, and P of them cover nk
__host__ __device__ inline int gg_part_stages(int nk, int P) { return ((nk + P - 1) / P + 1) & ~1; }

// How the tiles of a launch are walked: tiles [0, full) whole, tiles [full, total) in P parts each.
struct GgPlan {
    int total, full, P, nkp, units;
};
__host__ __device__ inline GgPlan gg_plan(int total, int grid, int nk, bool split, int max_units) {
    GgPlan pl;
    pl.total = total; pl.full = total; pl.P = 1; pl.nkp = nk;
    const int tail = total % grid;
    if (split && tail > 0 && 4 * tail <= grid) {
        int P = grid / tail;
        if (P > GG_MAX_PARTS) P = GG_MAX_PARTS;
        if (P > max_units / tail) P = max_units / tail;
        while (P > 1 && (gg_part_stages(nk, P) < GG_MIN_PART_STAGES || (P - 1) * gg_part_stages(nk, P) >= nk)) --P;
        if (P > 1) { pl.P = P; pl.full = total - tail; pl.nkp = gg_part_stages(nk, P); }
    }
    pl.units = pl.full + (total - pl.full) * pl.P;
    return pl;
}

// Where a packed weight column sits inside its aligned group of 32 rows of the packed matrix.  The MFMA leaves a lane
// with runs of FOUR consecutive rows of the weight operand (bf16 16x16: rows 4q .. 4q+3 of a tile for the lanes 16q ..
// 16q+15; fp8 32x32: rows 8Q + 4h .. + 3 for the register quad Q and the lanes 32h .. 32h+31).  The rows of a group are
// ordered so that two of a lane's runs are EIGHT consecutive output columns, which leave as one 16-byte store:
//   bf16: column 8q + 4t + v of the group (t = 0, 1: the group's two MFMA tiles) at row 16t + 4q + v;
//   fp8 : column 16P + 8h + 4t + v (P = 0, 1; quads 2P + t) at row 8 (2P + t) + 4h + v.
// Runs of four columns that start at a multiple of four stay runs of four rows.
template <bool FP8>
__host__ __device__ inline int gg_col_to_row32(int c) {  // c in [0, 32)
    if (FP8) return ((c >> 4) * 2 + ((c >> 2) & 1)) * 8 + ((c >> 3) & 1) * 4 + (c & 3);
    return ((c >> 2) & 1) * 16 + (c >> 3) * 4 + (c & 3);
}
template <bool FP8>
__host__ __device__ inline int gg_row_to_col32(int r) {  // the inverse
    if (FP8) return (r >> 4) * 16 + ((r >> 2) & 1) * 8 + ((r >> 3) & 1) * 4 + (r & 3);
    return ((r >> 2) & 3) * 8 + (r >> 4) * 4 + (r & 3);
}
template <bool FP8>
__host__ __device__ inline int gg_packed_row(int col) { return (col & ~31) | gg_col_to_row32<FP8>(col & 31); }
template <bool FP8>
__host__ __device__ inline int gg_packed_col(int row) { return (row & ~31) | gg_row_to_col32<FP8>(row & 31); }

// x * sigmoid(x) with the hardware reciprocal (1 ulp) instead of an IEEE division: the SwiGLU epilogue of a
// 128 x 128 wave tile evaluates this 8192 times per lane-row, and the division was most of its cost
// two fp32 -> packed bf16 (round to nearest even) in one hardware conversion
typedef __bf16 gg_bf16x2 __attribute__((ext_vector_type(2)));
typedef float gg_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t gg_pack_bf16(float lo, float hi) {
    const gg_f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, gg_bf16x2));
}
__device__ __forceinline__ float act_silu_fast(float x) { return x * __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }
__device__ __forceinline__ float act_silu(float x) { return x / (1.0f + __expf(-x)); }
__device__ __forceinline__ float act_gelu(float x) { return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f)); }

typedef float floatx4 __attribute__((ext_vector_type(4)));
// bf16: one 16x16x32 MFMA; lanes 16q .. 16q+15 hold K elements 8q .. 8q+7 (16 bytes) of rows 0 .. 15 of both operands
// (Z: the sum starts here -- the MFMA takes a constant zero as its C operand, so no accumulator is cleared beforehand)
template <bool Z = false>
__device__ __forceinline__ void mma_bf16_k32(floatx4& acc, const uint4& a, const uint4& b) {
    if constexpr (Z) {
        const floatx4 z = {0.f, 0.f, 0.f, 0.f};
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), z, 0, 0, 0);
    } else {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), acc, 0, 0, 0);
    }
}

// fp8: one 32x32x64 MFMA on 32 bytes of K per lane and operand (two 16-byte LDS chunks); both operands
// are split over the lanes and registers in the same way, so every k is multiplied exactly once
typedef int gg_i32x8 __attribute__((ext_vector_type(8)));
template <bool Z = false>
__device__ __forceinline__ void mma_fp8_k64(floatx16& acc, const uint4& a_lo, const uint4& a_hi, const uint4& b_lo, const uint4& b_hi) {
    const gg_i32x8 a = {(int)a_lo.x, (int)a_lo.y, (int)a_lo.z, (int)a_lo.w, (int)a_hi.x, (int)a_hi.y, (int)a_hi.z, (int)a_hi.w};
    const gg_i32x8 b = {(int)b_lo.x, (int)b_lo.y, (int)b_lo.z, (int)b_lo.w, (int)b_hi.x, (int)b_hi.y, (int)b_hi.z, (int)b_hi.w};
    // format selectors 0/0 = fp8 (e4m3) for both operands, no block scales
    if constexpr (Z) {
        const floatx16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, z, 0, 0, 0, 0, 0, 0);
    } else {
        acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc, 0, 0, 0, 0, 0, 0);
    }
}

// The same MFMA with block scales on the activation operand (the instruction's B: the kernels multiply transposed, weights
// as A).  For row r of the operand and block b of 32 k (b = 0: the first four registers of the lanes 0-31 and 32-63, i.e. k
// 0-15 and 16-31 of the step; b = 1: the other four registers), the scale is the E8M0 byte OPSEL of the scale register of
// lane 32 b + r (established with a one-wave probe on the chip); the weight operand takes 2^0 everywhere.
constexpr int GG_WSCALE = 64;
// ASMV: the instruction written out, accumulator in ordinary vector registers (the layout of eight waves per workgroup,
// where a wave's 256 registers hold accumulators and fragments alike).  Through the builtin, the compiler moves the scaled
// MFMAs of that layout across the scheduling fences that pin the K loop, bunches them, and spills accumulators and
// fragments inside the loop; a volatile asm statement stays where it is written.  The compiler does not know that the
// statement is an MFMA: what it would insert between such an instruction and a dependent one is added by hand where the
// accumulators are next read (GG_MFMA_SETTLE).
template <bool Z, int OPSEL, bool ASMV = false>
__device__ __forceinline__ void mma_fp8_k64_bs(floatx16& acc, const uint4& a_lo, const uint4& a_hi, const uint4& b_lo, const uint4& b_hi,
                                               int scale_b) {
    const gg_i32x8 a = {(int)a_lo.x, (int)a_lo.y, (int)a_lo.z, (int)a_lo.w, (int)a_hi.x, (int)a_hi.y, (int)a_hi.z, (int)a_hi.w};
    const gg_i32x8 b = {(int)b_lo.x, (int)b_lo.y, (int)b_lo.z, (int)b_lo.w, (int)b_hi.x, (int)b_hi.y, (int)b_hi.z, (int)b_hi.w};
    if constexpr (ASMV) {
        static_assert(!Z, "the written-out form accumulates");
        const int wsc = GG_WSCALE;
        if constexpr (OPSEL == 0)
            asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0]" : "+v"(acc) : "v"(a), "v"(b), "v"(wsc), "v"(scale_b));
        else
            asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,1,0]" : "+v"(acc) : "v"(a), "v"(b), "v"(wsc), "v"(scale_b));
        return;
    }
    // (the weight operand's scale byte is GG_WSCALE = 64, a constant the instruction can take without a register; the
    // activation side adds the 63 that are missing to 2^0 to its own bytes: the product of the two scales is what counts)
    if constexpr (Z) {
        const floatx16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, z, 0, 0, 0, GG_WSCALE, OPSEL, scale_b);
    } else {
        acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc, 0, 0, 0, GG_WSCALE, OPSEL, scale_b);
    }
}

// Block scale of the fp8 hidden activation: the smallest power of two X = 2^(byte - 127) with amax / X <= 448 (the largest
// e4m3 value), from the bits of amax >= 0: amax = m 2^p, 1 <= m < 2, fits when p - e < 8, or p - e = 8 and m <= 1.75 -- so
// byte = p + 127 - 8, one more when the mantissa exceeds that of 1.75; never below 0 (amax = 0, or tiny).  Integer work:
// the CPU checker computes the same byte from the same bits.
__host__ __device__ inline int gg_block_scale_byte(uint32_t amax_bits) {
    const int b = (int)((amax_bits + 0x1fffffu) >> 23) - 8;
    return b < 0 ? 0 : b;
}
// 1 / X as a float: 2^(127 - byte), exact (byte <= 247 for finite amax)
__host__ __device__ inline uint32_t gg_block_inv_bits(int byte) { return (uint32_t)(254 - byte) << 23; }

__device__ __forceinline__ int seg_of(const int* off, int n, int r) {
    int lo = 0, hi = n;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (off[mid] <= r) lo = mid; else hi = mid;
    }
    return lo;
}

// EPI_GATE: no activation, and every result row is multiplied by its row's gate (GemmParams::row_scale, one fp32
// multiplication before the rounding to bf16): the down projection of an expert whose rows return already weighted.
// (The fp8 kernels have a row scale as it is: a gate is folded into it by the caller.)
enum { EPI_NONE = 0, EPI_GELU = 1, EPI_SILU = 2, EPI_SWIGLU = 3, EPI_GATE = 4 };

// One output tile of the walk: group g, n tile nt, first row row0, rv valid rows (rv <= 0: none).
struct GgTile {
    int g, nt, row0, rv;
    int ks0, nks;   // first K stage and number of K stages this workgroup multiplies (the whole K range, or a part)
    int unit;       // part tile index in the partial-sum workspace, or -1 for a whole tile
};

// lin -> tile: group-major, 16-row bands, 16-column super-columns (see the XCD-aware walk above)
// DW (weight-gradient mode): every non-empty group has the same ceil(dw_rows / BM) x Nt tiles, rows [0, dw_rows) of its own
// output matrix; g_row_start then holds the groups' first K stages (set by the caller from it).
template <int BM, bool DW = false>
__device__ __forceinline__ GgTile gg_decode(const int* g_tile_start, const int* g_row_start, int E_l, int Nt, int S_rows, int lin,
                                            int dw_rows = 0) {
    const int g = seg_of(g_tile_start, E_l + 1, lin);
    const int cnt_g = DW ? dw_rows : g_row_start[g + 1] - g_row_start[g];
    const int Mt = (cnt_g + BM - 1) / BM;
    const int idx = lin - g_tile_start[g];
    const int band = idx / (SUP * Nt), rem = idx % (SUP * Nt);
    const int hr = min(SUP, Mt - band * SUP);
    const int sc = rem / (hr * SUP), rem2 = rem % (hr * SUP);
    const int wc = min(SUP, Nt - sc * SUP);
    const int mt = band * SUP + rem2 / wc;
    GgTile t;
    t.g = g;
    t.nt = sc * SUP + rem2 % wc;
    t.row0 = (DW ? 0 : g_row_start[g]) + mt * BM;
    t.rv = DW ? min(BM, cnt_g - mt * BM) : min(min(BM, cnt_g - mt * BM), S_rows - t.row0);
    return t;
}

// The tiles of a workgroup, in the order it walks them: round r of the persistent grid gives it tile r * stride + my.
// Decoding one costs a search and five integer divisions, so the workgroup decodes GG_TT of them at a time, one per
// thread, into a table in LDS; the walk itself is then one 16-byte LDS read per tile.
constexpr int GG_TT = 256;
template <int BM, bool SPLIT, bool DW>
__device__ __forceinline__ void gg_fill_table(int4* s_tiles, const int* g_tile_start, const int* g_row_start, int E_l, int Nt,
                                              int S_rows, const GgPlan& pl, int my, int stride, int round0, int dw_rows) {
    const int n = SPLIT ? pl.units - pl.full : pl.full;
    for (int i = threadIdx.x; i < GG_TT; i += blockDim.x) {
        const int lin = (round0 + i) * stride + my;
        int4 e = make_int4(0, 0, 0, 0);  // (g, nt, row0, rv); rv <= 0: nothing there
        if ((round0 + i) < (n + stride - 1) / stride && lin < n) {
            const GgTile t = gg_decode<BM, DW>(g_tile_start, g_row_start, E_l, Nt, S_rows, SPLIT ? pl.full + lin / pl.P : lin, dw_rows);
            e = make_int4(t.g, t.nt, t.row0, t.rv);
        }
        s_tiles[i] = e;
    }
}

// The tile of round `round` if the table holds it and it has rows (rv = 0 otherwise: the caller then takes the general
// walk below).  One LDS read; nothing is advanced, refilled or skipped.
template <bool SPLIT, bool DW>
__device__ __forceinline__ GgTile gg_peek(const int4* s_tiles, const int* g_row_start, const GgPlan& pl, int nk, int my, int stride,
                                          int round, int round0) {
    GgTile t;
    t.g = t.nt = t.row0 = 0;
    t.rv = 0;
    t.ks0 = 0; t.nks = nk; t.unit = -1;
    if (round < round0 + GG_TT) {  // (past the end of the walk the table holds empty entries)
        const int4 e = s_tiles[round - round0];
        t.g = __builtin_amdgcn_readfirstlane(e.x); t.nt = __builtin_amdgcn_readfirstlane(e.y);
        t.row0 = __builtin_amdgcn_readfirstlane(e.z); t.rv = max(__builtin_amdgcn_readfirstlane(e.w), 0);
        if constexpr (DW) {
            t.ks0 = g_row_start[t.g];
            t.nks = g_row_start[t.g + 1] - t.ks0;
        }
        if constexpr (SPLIT) {
            const int lin = round * stride + my;
            t.ks0 = (lin % pl.P) * pl.nkp;
            t.nks = min(pl.nkp, nk - t.ks0);
            t.unit = lin;
        }
    }
    return t;
}

// Next non-empty tile of this workgroup at or after round `round` (advanced past it); rv = 0 when there is none.
// round0 is the round the table starts at; the table is refilled (by the whole workgroup: every wave makes the same
// calls) when the walk leaves it.
template <int BM, bool SPLIT, bool DW>
__device__ __forceinline__ GgTile gg_walk(int4* s_tiles, const int* g_tile_start, const int* g_row_start, int E_l, int Nt, int S_rows,
                                          const GgPlan& pl, int nk, int my, int stride, int& round, int& round0, int dw_rows) {
    GgTile t;
    t.g = t.nt = t.row0 = 0;
    t.rv = 0;
    t.ks0 = 0; t.nks = nk; t.unit = -1;
    const int n = SPLIT ? pl.units - pl.full : pl.full;
    const int rounds = (n + stride - 1) / stride;
    while (round < rounds) {
        if (round >= round0 + GG_TT) {
            __syncthreads();  // (every wave has read what it needed of the old table)
            round0 = round;
            gg_fill_table<BM, SPLIT, DW>(s_tiles, g_tile_start, g_row_start, E_l, Nt, S_rows, pl, my, stride, round0, dw_rows);
            __syncthreads();
        }
        const int4 e = s_tiles[round - round0];
        const int lin = round * stride + my;
        ++round;
        const int rv = __builtin_amdgcn_readfirstlane(e.w);
        if (rv > 0) {
            t.g = __builtin_amdgcn_readfirstlane(e.x); t.nt = __builtin_amdgcn_readfirstlane(e.y);
            t.row0 = __builtin_amdgcn_readfirstlane(e.z); t.rv = rv;
            if constexpr (DW) {
                t.ks0 = g_row_start[t.g];
                t.nks = g_row_start[t.g + 1] - t.ks0;
            }
            if constexpr (SPLIT) {
                t.ks0 = (lin % pl.P) * pl.nkp;
                t.nks = min(pl.nkp, nk - t.ks0);
                t.unit = lin;
            }
            break;
        }
    }
    return t;
}


// ---- pieces of the main loop ---------------------------------------------------------------------
// HBM -> LDS, 16 bytes per lane, no register staging.  One instruction moves 16 tile rows of one ring
// stage (64 lanes x 16 B = 16 rows x 64 B); wave w of a round moves rows [w*16, w*16+16) of that round.
// Written as inline assembly to get the scalar-base + 32-bit-lane-offset form (the builtin expands to a
// 64-bit per-lane address); M0 holds the LDS byte address of the wave's 1 KB destination.
__device__ __forceinline__ void gg_dma16(const uint8_t* sbase, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0" : : "s"(sbase), "v"(voff), "s"(lds_addr) : "memory");
}

// The lane id read afresh (two instructions) where it is needed.  What the epilogue and the tile set-up derive from it
// is then computed there, once per tile, instead of being hoisted out of the tile loop as a dozen lane-constant
// invariants that occupy -- or spill -- registers across the whole K loop.
__device__ __forceinline__ int gg_lane_now() {
    int l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
    return l;
}

// One dword per lane, HBM -> LDS: lane l's value lands at lds_addr + 4 l.
__device__ __forceinline__ void gg_dma4(const uint8_t* sbase, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %1, %0" : : "s"(sbase), "v"(voff), "s"(lds_addr) : "memory");
}

// a wave-uniform value forced into scalar registers
__device__ __forceinline__ const uint8_t* gg_uniform(const uint8_t* p) {
    const uint64_t v = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const uint8_t*)(((uint64_t)hi << 32) | lo);
}

// s_waitcnt through the builtin (not inline asm) so that the compiler's own wait-count bookkeeping
// sees it.  gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14.
template <int VM, int LGKM>
__device__ __forceinline__ void gg_wait() {
    static_assert(VM >= 0 && VM <= 63 && LGKM >= 0 && LGKM <= 15, "wait counts");
    __builtin_amdgcn_s_waitcnt((VM & 15) | (7 << 4) | (LGKM << 8) | ((VM >> 4) << 14));
}

// NWM x 2 wave64s per workgroup; every wave owns a (BM/NWM) x 128 block of the tile.
//
// K moves through LDS in a ring of NRING stages of ROWB bytes per tile row.  A stage is one MFMA block
// (one 16x16x32 bf16 or 32x32x64 fp8 MFMA per pair of fragments).  The loads of stage s+4 go into the slot of
// stage s during block s -- every wave took the fragments of stage s into registers one block earlier -- spread
// over the block, so the load pipe sees a steady stream instead of a burst and every load has more than two
// blocks of MFMA work to land.
// SPLIT = false: the launch that takes whole tiles.  SPLIT = true: the launch that takes the tiles of an
// under-filled last round in parts of the K range and leaves fp32 partial sums in the workspace (GemmParams).
// BSA: the activation operand carries block scales (fp8 down projection: GemmParams::a_bscale), applied by the MFMAs.
// TRACE: the same kernel with time stamps (GemmParams::trace); product launches never use it.
template <int BM, int NWM, int EPI, bool FP8, bool SPLIT, bool DW = false, bool BSA = false, bool TRACE = false>
__global__ __launch_bounds__(NWM * 2 * WAVE, 1) void grouped_gemm_kernel(const GemmParams p) {
    static_assert(!TRACE || (!SPLIT && !DW), "time stamps: whole-tile forward launches only");
    [[maybe_unused]] int tr_tile = 0, tr_blk = 0;  // (TRACE) words written so far
#define GG_TRACE_TILE()                                                                                                    \
    do {                                                                                                                   \
        if constexpr (TRACE) {                                                                                             \
            if (threadIdx.x == 0 && tr_tile < GG_TRACE_TILE_WORDS) p.trace[(size_t)blockIdx.x * GG_TRACE_TILE_WORDS + tr_tile] = wall_clock64(); \
            ++tr_tile;                                                                                                     \
        }                                                                                                                  \
    } while (0)
    static_assert(!DW || (!SPLIT && !FP8 && EPI == EPI_NONE), "the weight-gradient mode is a plain bf16 GEMM");
    static_assert(!BSA || FP8, "block scales belong to the fp8 MFMA");
    constexpr bool VARK = SPLIT || DW;  // the K range differs from tile to tile
    constexpr bool PEEL = !VARK && !BSA;  // the tile's first two blocks written out apart (see below)
    constexpr bool QOUT = FP8 && EPI == EPI_SWIGLU && !SPLIT;  // the epilogue stores e4m3 codes and block scales
    constexpr int BN = GG_BN;
    constexpr int ES = FP8 ? 1 : 2;
    constexpr int NW = NWM * 2;                        // waves per workgroup
    // bf16: 16x16x32 MFMAs (4 accumulator registers each; under the power limit this shape sustains about
    // 15 % more than 32x32x16, which moves twice the accumulator bytes per flop); fp8: 32x32x64
    constexpr int MT = FP8 ? 32 : 16;                  // MFMA tile edge
    constexpr int CF = FP8 ? 2 : 1;                    // 16-byte LDS chunks per fragment and lane
    constexpr int TM = BM / (NWM * MT), TN = BN / (2 * MT);  // MFMA tiles per wave
    constexpr int NT = TM * TN;                        // MFMAs per K stage and wave
    constexpr int NRD = (TM + TN) * CF;                // fragment reads per K stage and wave
    constexpr int LR = NW * WROWS;                     // rows fetched per load round (16 per wave)
    constexpr int RA = BM / LR, RB = BN / LR;          // load rounds per stage
    constexpr int LPS = RA + RB;                       // HBM->LDS loads per lane per stage
    // Where the other instructions of a block sit.  bf16: a 16x16x32 MFMA covers only 16 cycles of other issue,
    // so no MFMA gets more than one: the fragment reads go behind every RSTEP-th MFMA of the first half of the
    // block (they must have landed when the block ends in the hand-over), the loads are spread evenly over the
    // whole block, behind other MFMAs where that fits (a steady stream to the load pipe: bunched at either end
    // of the block they cost 7 % more cycles).  fp8: a 32x32x64 MFMA covers 64 cycles and there are few of them;
    // two reads go behind each of the first MFMAs.
    constexpr int RPM = NRD > NT / 2 ? 2 : 1;                 // reads behind one MFMA
    constexpr int RFIRST = 0;                                 // first MFMA with a read behind it
    constexpr int RSTEP = (NT / 2) * RPM / NRD > 0 ? (NT / 2) * RPM / NRD : 1;  // MFMAs from one read group to the next
    constexpr int LFIRST = NT > LPS ? 1 : 0;                  // first MFMA with a load behind it
    constexpr int LSTEP = (NT - LFIRST) / LPS;                // MFMAs from one load to the next
    constexpr int ASLOT = BM * CHUNKS, BSLOT = BN * CHUNKS;  // uint4 per ring slot
    static_assert(TM * MT * NWM == BM && BM % LR == 0 && BN % LR == 0 && NT <= 64 && LSTEP >= 1 && LFIRST + LSTEP * (LPS - 1) < NT && RFIRST + RSTEP * ((NRD - 1) / RPM) < NT, "tile shape");
    static_assert(CHUNKS == 4 && NRING == 4, "the stage schedule below is written for 64-byte stages in four slots");

    __shared__ __align__(1024) uint4 sA[NRING * ASLOT];
    __shared__ __align__(1024) uint4 sB[NRING * BSLOT];
    __shared__ int g_tile_start[GG_MAXG + 1];
    __shared__ int g_row_start[GG_MAXG + 1];
    // what the epilogue needs from global memory per tile row / tile column (fp8 scales, the output row map)
    // (two copies, used by alternate tiles: a wave may enter the next tile while another is still in this one's epilogue)
    __shared__ __align__(16) float s_row_scale[2][BM];
    __shared__ __align__(16) float s_col_scale[2][BN];
    __shared__ int s_crow[2][BM];
    __shared__ int s_amap[BM];              // the NEXT tile's input rows (a_map), fetched while this one is multiplied
    // BSA: the block-scale bytes of the tile's rows for a PAIR of K stages (4 blocks of 32 k = one dword per row), two
    // copies: pairs alternate like the ring slots they travel with
    __shared__ uint32_t s_hsc[BSA ? 2 : 1][BSA ? BM : 1];
    __shared__ __align__(16) int4 s_tiles[GG_TT];
    static_assert(BM <= NWM * 2 * WAVE && BN <= NWM * 2 * WAVE, "one thread per tile row and per tile column");

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);  // the same, known to be wave-uniform (a scalar register)
    const int wm = wave >> 1, wn = wave & 1;
    const int Nt = p.Npad / BN;

    if (tid == 0) {
        int ts = 0, rs = 0;
        [[maybe_unused]] int dw_seen = 0;
        for (int g = 0; g < p.E_l; ++g) {
            g_tile_start[g] = ts;
            g_row_start[g] = rs;
            int c = max(p.cnt[g], 0);
            if constexpr (DW) {
                // tiles of the group's own dw_rows x N output; its K stages: the rows padded to 64 (two stages of 32)
                c = min(c, max(p.dw_src_rows - dw_seen, 0));
                dw_seen += c;
                ts += c > 0 ? ((p.dw_rows + BM - 1) / BM) * Nt : 0;
                rs += ((c + 63) / 64) * 2;
            } else {
                // (counts that claim more rows than the buffers hold are cut at S_rows: the host's bound on the number of
                // tiles, which decides whether the whole-tile launch is left out, counts on it)
                c = min(c, max(p.S_rows - rs, 0));
                ts += ((c + BM - 1) / BM) * Nt;
                rs += c;
            }
        }
        g_tile_start[p.E_l] = ts;
        g_row_start[p.E_l] = rs;
    }
    __syncthreads();
    const int nk = (p.K * ES) / ROWB;  // ring stages per tile; even (K * ES is a multiple of 2 * ROWB)
    const GgPlan plan = gg_plan(g_tile_start[p.E_l], (int)gridDim.x, nk, !DW && p.part_ws != nullptr, p.max_units);
    if (SPLIT && plan.P == 1) return;  // nothing was left over for this launch

    // XCD-aware position inside a round of gridDim.x tiles: workgroups b, b+8, b+16, ... share an L2.
    int my = blockIdx.x;
    if (gridDim.x == 256) {
        const int xcd = blockIdx.x & 7, l = blockIdx.x >> 3;
        my = (((xcd >> 1) * 4 + (l >> 3)) * SUP) + ((xcd & 1) * 8 + (l & 7));
    }

    // lane-constant pieces of the addressing.  A tile row is 4 chunks of 16 bytes; row r keeps logical
    // chunk c at position c ^ ((r >> 2) & 3), which makes both the 16-rows-per-instruction DMA writes
    // and the 128-bit fragment reads (rows = lane % 32) bank-conflict free.
    const int lrow = wave * WROWS + (lane >> 2);         // row inside a load round
    const int lchunk = (lane & 3) ^ ((lane >> 4) & 3);   // global 16-byte chunk this lane fetches
    const int fswz = (lane >> 2) & 3;                    // swizzle of the fragment row (tile rows start at multiples of 16)
    // first 16-byte chunk of the lane's fragment: bf16 lanes 16q .. 16q+15 take chunk q of rows 0 .. 15;
    // fp8 lanes 32h .. 32h+31 take chunks h and h + 2 of rows 0 .. 31 (both operands alike, so every k meets its partner):
    // the MFMA's first four operand registers of the two lane halves are then bytes 0-31 of the stage and the other four
    // bytes 32-63 -- the two blocks of 32 k that the scaled form of the instruction scales separately
    constexpr int FSTEP = FP8 ? 2 : 1;  // distance of a lane's second chunk
    const int fpos = (FP8 ? (lane >> 5) : (lane >> 4)) ^ fswz;
    const uint4* fa = sA + (wm * (BM / NWM) + (lane & (MT - 1))) * CHUNKS;
    const uint4* fb = sB + (wn * (BN / 2) + (lane & (MT - 1))) * CHUNKS;
    const uint32_t la0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)(sA + wave * WROWS * CHUNKS));
    const uint32_t lb0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)(sB + wave * WROWS * CHUNKS));

    const uint32_t ldk = (uint32_t)(p.K * ES);
    const size_t b_slab = (size_t)p.Npad * ROWB;  // packed weights are slab-major: [group][K slab][Npad rows][ROWB bytes]
    // per-round lane offsets into the weight slab (vector registers: no scalar address arithmetic per load)
    uint32_t b_off[RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) b_off[r] = (uint32_t)(r * LR + lrow) * ROWB + lchunk * 16;

#define GG_MAPROW_GLOBAL(t, l) p.a_map[(t).row0 + (l)]   /* the first tile: straight from memory */
#define GG_MAPROW_LDS(t, l) s_amap[(l)]                  /* later tiles: fetched into LDS one tile ahead */
#define GG_TILE_PTRS(t, Ab_, Bb_, aoff_, MAPROW_)                                                          \
    const uint8_t* Ab_ = (p.a_map ? p.A : p.A + (size_t)(t).row0 * p.K * ES) + (size_t)(t).ks0 * ROWB;      \
    const uint8_t* Bb_ = p.B + (DW ? (size_t)0 : (size_t)(t).g * p.Npad * p.K * ES) + (size_t)(t).nt * BN * ROWB + (size_t)(t).ks0 * b_slab; \
    uint32_t aoff_[RA];                                                                                     \
    const int ln_ = gg_lane_now();  /* lrow and lchunk again, derived per tile */                              \
    const int lrow_ = wave_s * WROWS + (ln_ >> 2);                                                            \
    const uint32_t lcb_ = (uint32_t)(((ln_ & 3) ^ ((ln_ >> 4) & 3)) * 16);                                     \
    _Pragma("unroll") for (int r = 0; r < RA; ++r) {                                                         \
        const int lr_ = max(min(r * LR + lrow_, (t).rv - 1), 0);  /* tile row this lane fetches, clamped */    \
        aoff_[r] = (uint32_t)(p.a_map ? max(MAPROW_(t, lr_), 0) : lr_) * ldk + lcb_;                       \
    }
    // load d (0 .. LPS-1) of one stage: A rounds first, then B rounds
#define GG_LD(d, ap_, bp_, aoff_, slot)                                                                       \
    do {                                                                                                      \
        if constexpr ((d) < RA) gg_dma16(ap_, aoff_[(d) < RA ? (d) : 0], la0 + ((slot) * ASLOT + (d) * LR * CHUNKS) * 16); \
        else gg_dma16(bp_, b_off[(d) >= RA ? (d) - RA : 0], lb0 + ((slot) * BSLOT + ((d) - RA) * LR * CHUNKS) * 16); \
    } while (0)
    // loads [first, first + count) of stage `st` (clamped to the last stage: the ring never holds data
    // of another tile, and a repeated load of the last stage lands in a slot nobody reads again)
#define GG_STAGE_PTRS(Ab_, Bb_, st, ap_, bp_, nks_)                                            \
    const int st_ = min((st), (nks_) - 1);                                                     \
    const uint8_t* ap_ = gg_uniform(Ab_ + (size_t)st_ * ROWB);                                 \
    const uint8_t* bp_ = gg_uniform(Bb_ + (size_t)st_ * b_slab);
#define GG_ISSUE_RANGE(Ab_, Bb_, aoff_, st, slot, first, count, nks_)                          \
    do {                                                                                       \
        GG_STAGE_PTRS(Ab_, Bb_, st, ap_i, bp_i, nks_)                                          \
        if constexpr ((first) + 0 < (first) + (count)) GG_LD((first) + 0 < LPS ? (first) + 0 : 0, ap_i, bp_i, aoff_, slot); \
        if constexpr ((first) + 1 < (first) + (count)) GG_LD((first) + 1 < LPS ? (first) + 1 : 0, ap_i, bp_i, aoff_, slot); \
        if constexpr ((first) + 2 < (first) + (count)) GG_LD((first) + 2 < LPS ? (first) + 2 : 0, ap_i, bp_i, aoff_, slot); \
        if constexpr ((first) + 3 < (first) + (count)) GG_LD((first) + 3 < LPS ? (first) + 3 : 0, ap_i, bp_i, aoff_, slot); \
        if constexpr ((first) + 4 < (first) + (count)) GG_LD((first) + 4 < LPS ? (first) + 4 : 0, ap_i, bp_i, aoff_, slot); \
        if constexpr ((first) + 5 < (first) + (count)) GG_LD((first) + 5 < LPS ? (first) + 5 : 0, ap_i, bp_i, aoff_, slot); \
        if constexpr ((first) + 6 < (first) + (count)) GG_LD((first) + 6 < LPS ? (first) + 6 : 0, ap_i, bp_i, aoff_, slot); \
        if constexpr ((first) + 7 < (first) + (count)) GG_LD((first) + 7 < LPS ? (first) + 7 : 0, ap_i, bp_i, aoff_, slot); \
        static_assert((count) <= 8, "GG_ISSUE_RANGE is unrolled for eight loads");             \
    } while (0)
    // what a tile has in flight before its first MFMA: its first four stages, one per ring slot
#define GG_PROLOGUE(Ab_, Bb_, aoff_, nks_)                    \
    do {                                                      \
        GG_SC_DMA(0, nks_, 0);                                \
        GG_ISSUE_RANGE(Ab_, Bb_, aoff_, 0, 0, 0, LPS, nks_);  \
        GG_ISSUE_RANGE(Ab_, Bb_, aoff_, 1, 1, 0, LPS, nks_);  \
        GG_SC_DMA(2, nks_, 2);                                \
        GG_ISSUE_RANGE(Ab_, Bb_, aoff_, 2, 2, 0, LPS, nks_);  \
        GG_ISSUE_RANGE(Ab_, Bb_, aoff_, 3, 3, 0, LPS, nks_);  \
    } while (0)

    // BSA: the block-scale bytes travel with the stages.  One dword per tile row holds the four scale bytes of a PAIR of
    // stages (2 x 64 bytes of K = 4 blocks of 32); it is requested, one per thread, straight into LDS with the loads of the
    // pair's even stage (same block, same ring slot: copy slot / 2), and read back by the lanes one block before the pair's
    // first MFMA.  sc_row0 / sc_rv / sc_ks0 describe the tile the loads currently point at (switched with Ab / Bb).
    [[maybe_unused]] int sc_row0 = 0, sc_rv = 1, sc_ks0 = 0;
    [[maybe_unused]] int sc[TM];
#define GG_SC_DMA(st, nks_, slot)                                                                                          \
    do {                                                                                                                   \
        if constexpr (BSA) {                                                                                               \
            if (wave_s * WAVE < BM) {                                                                                      \
                const int stc_ = min((st), (nks_) - 1);                                                                    \
                const int tid_c = wave_s * WAVE + gg_lane_now();                                                           \
                const uint32_t vo_ = (uint32_t)(sc_row0 + min(tid_c, sc_rv - 1)) * (uint32_t)p.bs_pitch +                  \
                                     (uint32_t)(((sc_ks0 + stc_) >> 1) << 2);                                              \
                gg_dma4(gg_uniform(p.a_bscale), vo_,                                                                       \
                        __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)(&s_hsc[(slot) >> 1][wave_s * WAVE]))); \
            }                                                                                                              \
        }                                                                                                                  \
    } while (0)
    // lane 32 h + r of a wave takes, for each of its row tiles, the dword of row r shifted so that byte 0 is the scale of
    // block h of the pair's even stage and byte 2 that of its odd stage (the MFMA's op_sel picks 0 or 2), each raised by
    // what the weight operand's constant scale byte lacks to 2^0.  One set of registers: a pair's dwords are read behind the
    // last MFMA of the pair before.
#define GG_SC_READ(SET_)                                                                                                   \
    do {                                                                                                                   \
        if constexpr (BSA) {                                                                                               \
            const int lnr_ = gg_lane_now();                                                                                \
            _Pragma("unroll") for (int i_ = 0; i_ < TM; ++i_)                                                               \
                sc[i_] = (int)(((s_hsc[SET_][(wave_s >> 1) * (BM / NWM) + i_ * MT + (lnr_ & 31)] >> ((lnr_ >> 5) * 8)) & 0x00ff00ffu) + \
                               (uint32_t)(127 - GG_WSCALE) * 0x00010001u);                                                 \
        }                                                                                                                  \
    } while (0)

    int round = 0, round0 = 0;
    gg_fill_table<BM, SPLIT, DW>(s_tiles, g_tile_start, g_row_start, p.E_l, Nt, p.S_rows, plan, my, (int)gridDim.x, 0, p.dw_rows);
    __syncthreads();
    GgTile cur = gg_walk<BM, SPLIT, DW>(s_tiles, g_tile_start, g_row_start, p.E_l, Nt, p.S_rows, plan, nk, my, (int)gridDim.x, round, round0, p.dw_rows);
    uint32_t a_off[RA];
    const uint8_t *Ab = p.A, *Bb = p.B;
    if (cur.rv > 0) {
        GG_TILE_PTRS(cur, Ab0, Bb0, a_off0, GG_MAPROW_GLOBAL);
        Ab = Ab0;
        Bb = Bb0;
#pragma unroll
        for (int r = 0; r < RA; ++r) a_off[r] = a_off0[r];
        sc_row0 = cur.row0; sc_rv = cur.rv; sc_ks0 = cur.ks0;
        GG_PROLOGUE(Ab, Bb, a_off, (VARK ? cur.nks : nk));
    }
    // The ring runs on from one tile into the next: the last four blocks of a tile refill their slots with the first
    // four stages of the NEXT tile (when the table has it at hand), its last block reads that tile's first fragments,
    // and the next tile then starts with everything in place -- no burst of 32 loads per lane with the matrix pipes
    // idle, no pair of barriers.  `pre` says that the tile at hand was prepared like that; phi is the ring slot of its
    // first stage (the ring is not realigned between tiles); tpar picks the copy of the epilogue data.
    uint4 fA0[TM * CF], fB0[TN * CF], fA1[TM * CF], fB1[TN * CF];
    bool pre = false;
    int phi = 0, tpar = 0;
    while (cur.rv > 0) {
        const int g = __builtin_amdgcn_readfirstlane(cur.g), nt = __builtin_amdgcn_readfirstlane(cur.nt);
        const int row0 = __builtin_amdgcn_readfirstlane(cur.row0), rv = __builtin_amdgcn_readfirstlane(cur.rv);
        const int nks = VARK ? __builtin_amdgcn_readfirstlane(cur.nks) : nk;
        const int unit = SPLIT ? __builtin_amdgcn_readfirstlane(cur.unit) : -1;

        typedef typename std::conditional<FP8, floatx16, floatx4>::type acc_t;
        acc_t acc[TM][TN];  // (not cleared where the MFMAs of the tile's first block start the sums)
        if constexpr (!PEEL) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int v = 0; v < (FP8 ? 16 : 4); ++v) acc[i][j][v] = 0.f;
        }

        // ---- One MFMA block per 64-byte stage.  Block s multiplies the fragments of stage s, reads those of
        // stage s+1 (all issued in the first half of the block, so they have landed when the block ends) and
        // refills slot s % 4, drained one block earlier, with stage s+4, its loads spread between the MFMAs
        // (a steady stream instead of a burst, each with three blocks of MFMA work to land); the hand-over at
        // its end waits for the wave's own loads of stage s+2 -- everything issued after them, stages s+3 and
        // s+4, may stay in flight -- and meets the other waves.  Loads past the end of the tile are clamped
        // to its last stage (straight-line code, constant wait counts); in the last block the "next
        // fragments" are whatever the next slot holds and are never used.  Every instruction is pinned by
        // scheduling fences: each read and each load is issued in the shadow of an MFMA.
        // fragment read R of the next stage: operand R / CF (activation rows first, then weight rows), chunk R % CF
#define GG_RD(R, NA_, NB_)                                                                               \
    do {                                                                                                 \
        constexpr int ro_ = (R) / CF, rh_ = (R) % CF;                                                    \
        if constexpr (ro_ < TM) NA_[ro_ * CF + rh_] = nfa_[ro_ * MT * CHUNKS + (fpos ^ (rh_ * FSTEP))];  \
        else NB_[(ro_ - TM) * CF + rh_] = nfb_[(ro_ - TM) * MT * CHUNKS + (fpos ^ (rh_ * FSTEP))];       \
    } while (0)
#define GG_ML(I, FA_, FB_, NA_, NB_, slot, Z_, EVEN_, SET_)                                                \
    do {                                                                                                 \
        if constexpr ((I) < NT) {                                                                        \
            /* boustrophedon over the wave's MFMA tiles: every instruction keeps one operand of the one before it */ \
            constexpr int pa_ = (I) / TN, pb_ = (pa_ & 1) ? TN - 1 - (I) % TN : (I) % TN;                \
            if constexpr (FP8 && BSA) mma_fp8_k64_bs<Z_, (EVEN_) ? 0 : 2, NWM == 4>(acc[pa_][pb_], FB_[2 * pb_], FB_[2 * pb_ + 1], FA_[2 * pa_], FA_[2 * pa_ + 1], sc[pa_]); \
            else if constexpr (FP8) mma_fp8_k64<Z_>(acc[pa_][pb_], FB_[2 * pb_], FB_[2 * pb_ + 1], FA_[2 * pa_], FA_[2 * pa_ + 1]); \
            else mma_bf16_k32<Z_>(acc[pa_][pb_], FB_[pb_], FA_[pa_]);                                    \
            __builtin_amdgcn_sched_barrier(0);                                                           \
            constexpr int ld_ = (I) >= LFIRST && ((I) - LFIRST) % LSTEP == 0 ? ((I) - LFIRST) / LSTEP : LPS;  /* load behind this MFMA */ \
            if constexpr (ld_ < LPS) GG_LD((ld_ < LPS ? ld_ : 0), ap_, bp_, a_off, slot);                \
            constexpr int r0_ = (I) >= RFIRST && ((I) - RFIRST) % RSTEP == 0 ? (((I) - RFIRST) / RSTEP) * RPM : NRD; /* first read */ \
            if constexpr (r0_ < NRD) GG_RD((r0_ < NRD ? r0_ : 0), NA_, NB_);                             \
            if constexpr (RPM > 1 && r0_ + 1 < NRD) GG_RD((r0_ + 1 < NRD ? r0_ + 1 : 0), NA_, NB_);      \
            __builtin_amdgcn_sched_barrier(0);                                                           \
        }                                                                                                \
    } while (0)
#define GG_ML8(I, FA_, FB_, NA_, NB_, slot, Z_, E_, S_)                                                          \
    GG_ML((I) + 0, FA_, FB_, NA_, NB_, slot, Z_, E_, S_); GG_ML((I) + 1, FA_, FB_, NA_, NB_, slot, Z_, E_, S_);           \
    GG_ML((I) + 2, FA_, FB_, NA_, NB_, slot, Z_, E_, S_); GG_ML((I) + 3, FA_, FB_, NA_, NB_, slot, Z_, E_, S_);           \
    GG_ML((I) + 4, FA_, FB_, NA_, NB_, slot, Z_, E_, S_); GG_ML((I) + 5, FA_, FB_, NA_, NB_, slot, Z_, E_, S_);           \
    GG_ML((I) + 6, FA_, FB_, NA_, NB_, slot, Z_, E_, S_); GG_ML((I) + 7, FA_, FB_, NA_, NB_, slot, Z_, E_, S_)
    // SET_: which copy of the block scales (BSA) the stage's pair uses: slot / 2, as a literal (0 where the slot is a run-time value: no BSA there)
#define GG_STAGE(FA_, FB_, NA_, NB_, SL, EVEN_, s, last, Z_, SET_)                                                \
    do {                                                                                                 \
        if constexpr (EVEN_) { /* (a block in an even slot) */                                           \
            /* from block nks - 4 on the loads fetch the next tile, if it is at hand; not in a tile's first block: the  \
               row map that the tile's top requested must have landed and been handed over (one block end at least) */ \
            if ((s) == nks - 4 && (s) > 0) {                                                             \
                const GgTile pk_ = gg_peek<SPLIT, DW>(s_tiles, g_row_start, plan, nk, my, (int)gridDim.x, round, round0); \
                if (pk_.rv > 0) {                                                                        \
                    GG_TILE_PTRS(pk_, Ab_s, Bb_s, a_off_s, GG_MAPROW_LDS);                               \
                    Ab = Ab_s;                                                                           \
                    Bb = Bb_s;                                                                           \
                    _Pragma("unroll") for (int r = 0; r < RA; ++r) a_off[r] = a_off_s[r];                \
                    kbase = nks;                                                                         \
                    nks_ld = VARK ? pk_.nks : nk;                                                        \
                    seam = true;                                                                         \
                    sc_row0 = pk_.row0; sc_rv = pk_.rv; sc_ks0 = pk_.ks0;                                \
                }                                                                                        \
            }                                                                                            \
            /* (the scale dwords of the pair whose even stage this block requests) */                   \
            GG_SC_DMA((s) + 4 - kbase, nks_ld, SET_ * 2);                                                \
        }                                                                                                \
        GG_STAGE_PTRS(Ab, Bb, (s) + 4 - kbase, ap_, bp_, nks_ld)                                         \
        const uint4* nfa_ = fa + (((SL) + 1) & 3) * ASLOT;                                               \
        const uint4* nfb_ = fb + (((SL) + 1) & 3) * BSLOT;                                               \
        /* (written-out MFMAs: two wait states between the vector instructions above and an MFMA that reads their results) */ \
        if constexpr (BSA && NWM == 4) asm volatile("s_nop 1");                                          \
        __builtin_amdgcn_sched_barrier(0);                                                               \
        GG_ML8(0, FA_, FB_, NA_, NB_, SL, Z_, EVEN_, SET_); GG_ML8(8, FA_, FB_, NA_, NB_, SL, Z_, EVEN_, SET_);   \
        GG_ML8(16, FA_, FB_, NA_, NB_, SL, Z_, EVEN_, SET_); GG_ML8(24, FA_, FB_, NA_, NB_, SL, Z_, EVEN_, SET_); \
        GG_ML8(32, FA_, FB_, NA_, NB_, SL, Z_, EVEN_, SET_); GG_ML8(40, FA_, FB_, NA_, NB_, SL, Z_, EVEN_, SET_); \
        GG_ML8(48, FA_, FB_, NA_, NB_, SL, Z_, EVEN_, SET_); GG_ML8(56, FA_, FB_, NA_, NB_, SL, Z_, EVEN_, SET_); \
        /* an odd block ends a pair: the next pair's scale dwords, from the other copy, behind its last MFMA */ \
        if constexpr (!(EVEN_)) GG_SC_READ(1 - SET_);                                                    \
        if (!(last) || seam) { /* (the last block hands over too when the next tile's stages are behind it) */ \
            gg_wait<2 * LPS, 0>();                                                                       \
            __builtin_amdgcn_s_barrier();                                                                \
        }                                                                                                \
        if constexpr (TRACE) {                                                                           \
            if (blockIdx.x == 0 && threadIdx.x == 0 && tr_blk < GG_TRACE_BLOCK_WORDS)                    \
                p.trace[(size_t)gridDim.x * GG_TRACE_TILE_WORDS + tr_blk] = wall_clock64();              \
            ++tr_blk;                                                                                    \
        }                                                                                                \
    } while (0)
        GG_TRACE_TILE();
        int kbase = 0, nks_ld = nks;  // the loads of block s fetch stage s + 4 - kbase of the tile (Ab, Bb, a_off) point to
        bool seam = false;            // ... which is the next tile from block nks - 4 on
        {
            if (!pre) {
                // the four stages of this tile were requested before the previous tile's epilogue (or above, for
                // the first tile); the epilogue's stores sit behind them in the same counter, so wait for
                // everything
                gg_wait<0, 15>();
                __syncthreads();
            }
            if (p.a_map) {
                // the input rows of the NEXT tile, one per thread, straight into LDS: the switch to the next tile inside
                // this tile's K loop then reads them from there instead of waiting for memory
                const GgTile pk = gg_peek<SPLIT, DW>(s_tiles, g_row_start, plan, nk, my, (int)gridDim.x, round, round0);
                if (pk.rv > 0 && wave_s * WAVE < BM) {
                    const int tid_a = wave_s * WAVE + gg_lane_now();
                    gg_dma4(gg_uniform((const uint8_t*)(p.a_map + pk.row0)), (uint32_t)min(tid_a, pk.rv - 1) * 4u,
                            __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)(s_amap + wave_s * WAVE)));
                }
            }
            if constexpr (!SPLIT) {
                // What the epilogue needs from global memory per tile row / column (fp8 scales, the output row map) is
                // requested here, straight into LDS, one value per thread (into the copy the previous tile does not
                // use): the loads land during the first K stages (they are older than every load the K loop waits
                // for), and no epilogue waits for a memory round trip.  No register holds anything across the K loop.
                const int lane_t = gg_lane_now(), tid_t = wave_s * WAVE + lane_t;  // (a fresh lane id: nothing kept live for this)
                const uint32_t t4 = (uint32_t)min(tid_t, rv - 1) * 4u;
                if (wave_s * WAVE < BM) {
                    if ((FP8 || EPI == EPI_GATE) && (!BSA || p.row_scale))  // (BSA: the rows carry no scale of their own; a gate, if any)
                        gg_dma4(gg_uniform((const uint8_t*)(p.row_scale + row0)), t4,
                                __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)(s_row_scale[tpar] + wave_s * WAVE)));
                    if (p.c_map)
                        gg_dma4(gg_uniform((const uint8_t*)(p.c_map + row0)), t4,
                                __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)(s_crow[tpar] + wave_s * WAVE)));
                }
                if (FP8 && wave_s * WAVE < BN) {
                    const int pc = gg_packed_col<true>(nt * BN + tid_t);  // packed column of the launch behind this row of the weight tile; the lanes 32..63 of a wave hold up columns
                    int col = EPI == EPI_SWIGLU ? (pc / 64) * 32 + pc % 32 : pc;
                    col = col < p.N ? col : 0;  // (columns past N are never stored: any valid scale will do)
                    const uint32_t lds_cs = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)(s_col_scale[tpar] + wave_s * WAVE));
                    const uint32_t c4 = (uint32_t)col * 4u;
                    if (EPI == EPI_SWIGLU && lane_t >= 32) gg_dma4(gg_uniform((const uint8_t*)(p.col_scale2 + (size_t)g * p.ncs)), c4, lds_cs);
                    else gg_dma4(gg_uniform((const uint8_t*)(p.col_scale + (size_t)g * p.ncs)), c4, lds_cs);
                }
            }
            if (!pre) {
                const uint4* fa0 = fa + phi * ASLOT;
                const uint4* fb0 = fb + phi * BSLOT;
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int h = 0; h < CF; ++h) fA0[i * CF + h] = fa0[i * MT * CHUNKS + (fpos ^ (h * FSTEP))];
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int h = 0; h < CF; ++h) fB0[j * CF + h] = fb0[j * MT * CHUNKS + (fpos ^ (h * FSTEP))];
                GG_SC_READ(0);  // (a tile that starts here starts in slot 0)
                // the first slot is refilled from the first block on: every wave must hold its stage-0 fragments first
                gg_wait<63, 0>();
                __syncthreads();
            }
            // The blocks are written out for the slots 0 .. 3; a tile whose first stage lies in slot 2 (phi = 2: the
            // tiles before it left the ring there) enters at the third.  nk >= 2 and even.
            if constexpr (PEEL) {
                // The tile's first two blocks are written out apart, with the slot as a run-time value: the MFMAs of the
                // very first start the sums (constant zero as their C operand), so that no accumulator has to be cleared
                // between two tiles.  (Not where the stage count varies from tile to tile: the register allocation of
                // those instantiations does not survive it.)
                const int phi_s = __builtin_amdgcn_readfirstlane(phi);
                GG_STAGE(fA0, fB0, fA1, fB1, phi_s, true, 0, false, true, 0);
                GG_STAGE(fA1, fB1, fA0, fB0, phi_s + 1, false, 1, 2 >= nks, false, 0);
                int ks = phi_s ? 2 : 0;             // phi = 0: on with the slots 2, 3 (the first half of the loop body is
                const int kmin = phi_s ? 2 : 4;     // skipped once); phi = 2: with the slots 0, 1
                while (ks < nks) {
                    if (ks >= kmin) {
                        GG_STAGE(fA0, fB0, fA1, fB1, 0, true, ks, false, false, 0);
                        GG_STAGE(fA1, fB1, fA0, fB0, 1, false, ks + 1, ks + 2 >= nks, false, 0);
                    }
                    if (ks + 2 < nks) {
                        GG_STAGE(fA0, fB0, fA1, fB1, 2, true, ks + 2, false, false, 1);
                        GG_STAGE(fA1, fB1, fA0, fB0, 3, false, ks + 3, ks + 4 >= nks, false, 1);
                    }
                    ks += 4;
                }
            } else {
                int ks = -phi;
                do {
                    if (ks >= 0) {
                        GG_STAGE(fA0, fB0, fA1, fB1, 0, true, ks, false, false, 0);
                        GG_STAGE(fA1, fB1, fA0, fB0, 1, false, ks + 1, ks + 2 >= nks, false, 0);
                    }
                    if (ks + 2 < nks) {
                        GG_STAGE(fA0, fB0, fA1, fB1, 2, true, ks + 2, false, false, 1);
                        GG_STAGE(fA1, fB1, fA0, fB0, 3, false, ks + 3, ks + 4 >= nks, false, 1);
                    }
                    ks += 4;
                } while (ks < nks);
            }
        }
#undef GG_STAGE
#undef GG_ML8
#undef GG_ML
#undef GG_RD

        if constexpr (BSA && NWM == 4) {
            // the last MFMAs of the tile were written out as asm (see mma_fp8_k64_bs): the wait states the compiler would put
            // between an MFMA and the first read of its result by another kind of instruction (18 for this shape)
            asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
        }
        // ---- next tile: decode it and request its first stages now (every slot is free once all waves
        // have passed the barrier: the last fragments of this tile are already in registers)
        // (when the K loop has switched over, the walk only confirms what the look-ahead saw)
        GG_TRACE_TILE();
        const GgTile nxt = gg_walk<BM, SPLIT, DW>(s_tiles, g_tile_start, g_row_start, p.E_l, Nt, p.S_rows, plan, nk, my, (int)gridDim.x, round, round0, p.dw_rows);
        if (!seam && nxt.rv > 0) {
            GG_TILE_PTRS(nxt, Ab_n, Bb_n, a_off_n, GG_MAPROW_GLOBAL);
            Ab = Ab_n;
            Bb = Bb_n;
#pragma unroll
            for (int r = 0; r < RA; ++r) a_off[r] = a_off_n[r];
            sc_row0 = nxt.row0; sc_rv = nxt.rv; sc_ks0 = nxt.ks0;
            __syncthreads();
            GG_PROLOGUE(Ab, Bb, a_off, (VARK ? nxt.nks : nk));
        }
        const int phi_n = seam ? ((phi + nks) & 3) : 0;

        // ---- a part of a tile: its fp32 partial sums go to the workspace as they are (tile row major, 256
        // columns; the lane's runs of four columns as 16-byte stores); the reduction kernel does the rest
        if constexpr (SPLIT) {  // (every tile of this instantiation is a part; the epilogue below is the other one's)
            float* wsT = p.part_ws + (size_t)unit * (BM * BN);
            constexpr int NQp = FP8 ? 4 : 1;
            const int lane_p = gg_lane_now(), rbase_p = (wave_s >> 1) * (BM / NWM);
            const int clp = FP8 ? (lane_p >> 5) * 4 : (lane_p >> 4) * 4;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int r = rbase_p + i * MT + (lane_p & (MT - 1));
#pragma unroll
                for (int j = 0; j < TN; ++j) {
#pragma unroll
                    for (int q = 0; q < NQp; ++q) {
                        const int c = wn * (BN / 2) + j * MT + 8 * q + clp;
                        const float4 v = make_float4(acc[i][j][4 * q + 0], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                                                     acc[i][j][4 * q + 3]);
                        if (r < rv) *(float4*)(wsT + (size_t)r * BN + c) = v;
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            cur = nxt;
            pre = seam;
            phi = phi_n;
            tpar ^= 1;
            continue;
        }

        // ---- epilogue: acc -> (scales) -> activation -> bf16 -> C
        // acc(i,j) holds the TRANSPOSED MT x MT product (weights as the MFMA A operand, activations as B):
        // a lane owns one token row of the tile and runs of four consecutive rows of the weight tile
        //   bf16 (16x16): token row l % 16, weight rows 4 * (l / 16) + v, v = 0..3
        //   fp8  (32x32): token row l % 32, weight rows 8 * q + 4 * (l / 32) + v for the four register quads q
        // and the rows of a group of 32 packed columns are ordered (gg_col_to_row32) so that two of those runs are
        // eight consecutive output columns -> 16-byte stores.
        // SwiGLU: packed columns alternate gate / up in groups of 32, so a gate group and its up group lie
        // 32 packed columns apart and land on output column (packed column of the gate group) / 2 + ... .
        bf16_t* C = (bf16_t*)p.C;
        constexpr int GT = 32 / MT;                  // MFMA tiles per group of 32 packed columns
        constexpr int NG = TN / GT;                  // groups per wave (its 128 packed columns)
        constexpr int NU = FP8 ? 2 : 1;              // 16-byte stores per lane and group
        // (the lane-derived constants of the epilogue are derived here, once per tile, from a fresh read of the lane id)
        const int lane_e = gg_lane_now(), rbase_e = (wave_s >> 1) * (BM / NWM), cbase_e = (wave_s & 1) * (BN / 2);
        const int lsub = FP8 ? (lane_e >> 5) : (lane_e >> 4);  // which of the lanes that share a tile row this one is
        // What the tile's top requested into LDS (scales, row map) is behind two block ends of the K loop at least -- the
        // second one has waited for it in every wave -- unless the tile has only two stages:
        if (nks < 4 && (FP8 || EPI == EPI_GATE || p.c_map)) {
            gg_wait<0, 15>();
            __syncthreads();
        }
        // fp8 with bf16 output: a lane stores to TWO rows of a row tile (its accumulators change lanes first, below);
        // bf16, and fp8 with quantised output: to its own
        constexpr int NR = (FP8 && !QOUT) ? 2 : 1;
        bool ok[TM][NR];
        bf16_t* crow[TM][NR];
        float rs[TM];
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            rs[i] = 1.f;
            if constexpr (FP8 || EPI == EPI_GATE) {
                if (!BSA || p.row_scale) rs[i] = s_row_scale[tpar][rbase_e + i * MT + (lane_e & (MT - 1))];  // (of the row it computed)
            }
#pragma unroll
            for (int h = 0; h < NR; ++h) {
                const int r = rbase_e + i * MT + ((FP8 && !QOUT) ? (lane_e & 15) + 16 * h : (lane_e & (MT - 1)));
                ok[i][h] = r < rv && !(TRACE && (p.trace_flags & 1));
                const size_t grow = (size_t)(row0 + (ok[i][h] ? r : 0));
                const int crow_i = p.c_map ? s_crow[tpar][r] : 0;
                ok[i][h] = ok[i][h] && crow_i >= 0;  // a negative map entry: the row has no place in the output
                // (quantised output: C holds one-byte codes, addressed below from the same row index)
                crow[i][h] = C + (p.c_map ? (size_t)max(crow_i, 0) : grow) * (QOUT ? (size_t)1 : (size_t)p.ldc) + (DW ? (size_t)g * p.c_group_stride : (size_t)0);
            }
        }
#pragma unroll
        for (int o = 0; o < TM * NG; ++o) {
            // fp8: column groups outermost; bf16: row tiles outermost, so that the stores of one row tile fill whole
            // cache lines back to back (the other order wrote 50 % more bytes to memory: lines left the L2
            // half written)
            const int i = FP8 ? o % TM : o / NG, jg = FP8 ? o / TM : o % NG;
            if constexpr (EPI == EPI_SWIGLU) {
                if (jg % 2 == 1) continue;  // an up group: consumed together with its gate group
            }
            const int pcol = nt * BN + cbase_e + jg * 32;  // first packed column of the group
            const int colg = EPI == EPI_SWIGLU ? (pcol / 64) * 32 : pcol;  // its first output column
            [[maybe_unused]] uint4 pk[2];  // fp8: the lane's two 16-byte units of the group, stored after they changed lanes
            [[maybe_unused]] float xq[2][8];  // quantised output: the lane's sixteen values of the group's block of 32 columns
#pragma unroll
            for (int u = 0; u < NU; ++u) {
                // the lane's eight consecutive columns: two runs of four accumulators (bf16: the group's two tiles;
                // fp8: the register quads 2u and 2u + 1 of the group's one tile)
                const int col = colg + (FP8 ? 16 * u : 0) + 8 * lsub;
                float x[8];
                [[maybe_unused]] float pre_g[8], pre_u[8];  // bf16 kernels asked to keep them: the values before the activation
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const int j = FP8 ? jg : jg * GT + t;       // MFMA tile of the run
                    const int qd = FP8 ? 2 * u + t : 0;         // its register quad
                    const int ju = j + GT;                      // SwiGLU: the up tile (32 packed columns further)
                    float cg[4] = {1.f, 1.f, 1.f, 1.f}, cu[4] = {1.f, 1.f, 1.f, 1.f};
                    if constexpr (FP8) {
                        // channel scales by row of the weight tile (an LDS read: cheap enough to repeat for every row tile)
                        const int tc = cbase_e + j * MT + 8 * qd + 4 * lsub;
                        const float4 s0 = *(const float4*)(s_col_scale[tpar] + tc);
                        cg[0] = s0.x; cg[1] = s0.y; cg[2] = s0.z; cg[3] = s0.w;
                        if constexpr (EPI == EPI_SWIGLU) {
                            const float4 s1 = *(const float4*)(s_col_scale[tpar] + tc + 32);
                            cu[0] = s1.x; cu[1] = s1.y; cu[2] = s1.z; cu[3] = s1.w;
                        }
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float v = acc[i][j][4 * qd + e];
                        if constexpr (FP8) v *= cg[e] * rs[i];
                        if constexpr (!FP8 && EPI == EPI_GATE) v *= rs[i];
                        if constexpr (!FP8 && EPI != EPI_NONE && EPI != EPI_GATE) pre_g[4 * t + e] = v;
                        if constexpr (EPI == EPI_SWIGLU) {
                            float uv = acc[i][ju % TN][4 * qd + e];
                            if constexpr (FP8) uv *= cu[e] * rs[i];
                            if constexpr (!FP8) pre_u[4 * t + e] = uv;
                            v = act_silu_fast(v) * uv;
                        }
                        if constexpr (EPI == EPI_GELU) v = act_gelu(v);
                        if constexpr (EPI == EPI_SILU) v = act_silu_fast(v);
                        x[4 * t + e] = v;
                    }
                }
                if constexpr (QOUT) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) xq[u][e] = x[e];
                    continue;
                }
                uint4 o4;
                o4.x = gg_pack_bf16(x[0], x[1]);
                o4.y = gg_pack_bf16(x[2], x[3]);
                o4.z = gg_pack_bf16(x[4], x[5]);
                o4.w = gg_pack_bf16(x[6], x[7]);
                if constexpr (FP8) {
                    pk[u] = o4;
                } else if (ok[i][0] && col < p.N) {
                    *(uint4*)(crow[i][0] + col) = o4;
                    if constexpr (EPI != EPI_NONE && EPI != EPI_GATE) {
                        if (p.C2) {
                            // same row, in a matrix whose rows are as long (SwiGLU: twice as long, packed column order)
                            constexpr int W2 = EPI == EPI_SWIGLU ? 2 : 1;
                            bf16_t* r2 = (bf16_t*)p.C2 + (size_t)(crow[i][0] - C) * W2 + (EPI == EPI_SWIGLU ? pcol + 8 * lsub : col);
                            uint4 g4;
                            g4.x = gg_pack_bf16(pre_g[0], pre_g[1]); g4.y = gg_pack_bf16(pre_g[2], pre_g[3]);
                            g4.z = gg_pack_bf16(pre_g[4], pre_g[5]); g4.w = gg_pack_bf16(pre_g[6], pre_g[7]);
                            *(uint4*)r2 = g4;
                            if constexpr (EPI == EPI_SWIGLU) {
                                uint4 u4;
                                u4.x = gg_pack_bf16(pre_u[0], pre_u[1]); u4.y = gg_pack_bf16(pre_u[2], pre_u[3]);
                                u4.z = gg_pack_bf16(pre_u[4], pre_u[5]); u4.w = gg_pack_bf16(pre_u[6], pre_u[7]);
                                *(uint4*)(r2 + 32) = u4;
                            }
                        }
                    }
                }
            }
            if constexpr (QOUT) {
                // The group is one block of 32 output columns of the hidden activation: the lane holds 16 of its values
                // (columns 8 lsub .. + 7 and 16 + 8 lsub .. + 7), the lane 32 further the other 16.  Block scale = the
                // smallest power of two under which the block's largest magnitude fits e4m3; codes = the values divided by
                // it (exact), rounded to e4m3; the two lanes trade a run of 8 codes each, so that each stores 16 contiguous
                // bytes of its row; one lane of the pair stores the scale byte.
                float am = 0.f;
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int e = 0; e < 8; ++e) am = fmaxf(am, fabsf(xq[u][e]));
                {
                    const auto sw_ = __builtin_amdgcn_permlane32_swap(__float_as_uint(am), __float_as_uint(am), false, false);
                    am = fmaxf(__uint_as_float(sw_[0]), __uint_as_float(sw_[1]));
                }
                const int sbyte = gg_block_scale_byte(__float_as_uint(am));
                const float inv = __uint_as_float(gg_block_inv_bits(sbyte));
                uint32_t cd[2][2];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    int lo = 0, hi = 0;
                    lo = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(xq[u][0], inv), __fmul_rn(xq[u][1], inv), lo, false);
                    lo = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(xq[u][2], inv), __fmul_rn(xq[u][3], inv), lo, true);
                    hi = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(xq[u][4], inv), __fmul_rn(xq[u][5], inv), hi, false);
                    hi = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(xq[u][6], inv), __fmul_rn(xq[u][7], inv), hi, true);
                    cd[u][0] = (uint32_t)lo;
                    cd[u][1] = (uint32_t)hi;
                }
                // lanes 0-31 keep their first run and take the partner's first run (columns 0-15 of the block), lanes 32-63
                // take the partner's second run and keep their own (columns 16-31)
                const auto s0_ = __builtin_amdgcn_permlane32_swap(cd[0][0], cd[1][0], false, false);
                const auto s1_ = __builtin_amdgcn_permlane32_swap(cd[0][1], cd[1][1], false, false);
                const uint4 codes = make_uint4(s0_[0], s1_[0], s0_[1], s1_[1]);
                const int col = colg + 16 * lsub;
                if (ok[i][0] && col < p.N) {
                    uint8_t* qrow = (uint8_t*)p.C + (size_t)(crow[i][0] - C) * p.ldc;
                    *(uint4*)(qrow + col) = codes;
                    if (lsub == 0) p.c_bscale[(size_t)(crow[i][0] - C) * p.bs_pitch + colg / 32] = (uint8_t)sbyte;
                }
            } else if constexpr (FP8) {
                // A lane holds 16 bytes of each half of its row's 64 (columns 8 lsub .. and 16 + 8 lsub ..) and the lane 16
                // further the same of the row 16 further.  They trade one half each (v_permlane16_swap: lanes 16-31 and
                // 48-63 of the first operand against lanes 0-15 and 32-47 of the second), after which the first operand
                // holds whole 64-byte segments of rows 0-15 of the row tile and the second those of rows 16-31: a store
                // instruction then covers 16 rows instead of 32 -- the store path's cost follows the number of row
                // segments per instruction, not the bytes.
#define GG_SWAP16(a_, b_)                                                          \
    do {                                                                           \
        const auto sw_ = __builtin_amdgcn_permlane16_swap((a_), (b_), false, false); \
        (a_) = sw_[0];                                                             \
        (b_) = sw_[1];                                                             \
    } while (0)
                GG_SWAP16(pk[0].x, pk[1].x);
                GG_SWAP16(pk[0].y, pk[1].y);
                GG_SWAP16(pk[0].z, pk[1].z);
                GG_SWAP16(pk[0].w, pk[1].w);
#undef GG_SWAP16
                const int col = colg + 16 * ((lane_e >> 4) & 1) + 8 * lsub;
                if (col < p.N) {
                    if (ok[i][0]) *(uint4*)(crow[i][0] + col) = pk[0];
                    if (ok[i][NR - 1]) *(uint4*)(crow[i][NR - 1] + col) = pk[1];
                }
            }
            // keep the accumulator read-out of one group from being hoisted over the previous group's stores
            // (that would need every accumulator in a VGPR at once)
            __builtin_amdgcn_sched_barrier(0);
        }
        GG_TRACE_TILE();
        cur = nxt;
        pre = seam;
        phi = phi_n;
        tpar ^= 1;
    }
#undef GG_TRACE_TILE
#undef GG_TILE_PTRS
#undef GG_MAPROW_GLOBAL
#undef GG_MAPROW_LDS
#undef GG_LD
#undef GG_STAGE_PTRS
#undef GG_ISSUE_RANGE
#undef GG_PROLOGUE
#undef GG_SC_DMA
#undef GG_SC_READ
}

// ---- second half of a K-split tile: add its parts in part order, then the epilogue of the GEMM kernel ------------
// Same tile tables and the same plan as the GEMM launch it follows (gemm_grid = that launch's grid).  A block takes
// BM / GG_RED_SLABS rows of one split tile (many small blocks: the partial sums of a few tiles are tens of MB); a thread takes four consecutive output columns of a row (for SwiGLU the gate
// columns and, 32 packed columns further, their up columns).
template <int BM, int EPI, bool FP8>
__global__ __launch_bounds__(256) void gg_reduce_parts_kernel(const GemmParams p, int gemm_grid) {
    constexpr int BN = GG_BN;
    constexpr int ES = FP8 ? 1 : 2;
    constexpr int RSL = GG_RED_SLABS;  // row slabs (blocks) per tile
    __shared__ int g_tile_start[GG_MAXG + 1];
    __shared__ int g_row_start[GG_MAXG + 1];
    const int Nt = p.Npad / BN;
    if (threadIdx.x == 0) {
        int ts = 0, rs = 0;
        for (int g = 0; g < p.E_l; ++g) {
            g_tile_start[g] = ts;
            g_row_start[g] = rs;
            const int c = min(max(p.cnt[g], 0), max(p.S_rows - rs, 0));  // (clamped like the GEMM launch clamps it)
            ts += ((c + BM - 1) / BM) * Nt;
            rs += c;
        }
        g_tile_start[p.E_l] = ts;
        g_row_start[p.E_l] = rs;
    }
    __syncthreads();
    const int nk = (p.K * ES) / ROWB;
    const GgPlan plan = gg_plan(g_tile_start[p.E_l], gemm_grid, nk, true, p.max_units);
    if (plan.P == 1) return;
    const int ti = blockIdx.x / RSL, slab = blockIdx.x % RSL;
    if (ti >= plan.total - plan.full) return;
    const GgTile t = gg_decode<BM>(g_tile_start, g_row_start, p.E_l, Nt, p.S_rows, plan.full + ti);
    if (t.rv <= 0) return;
    const float* ws = p.part_ws + (size_t)ti * plan.P * (BM * BN);
    constexpr int OC4 = (EPI == EPI_SWIGLU ? BN / 2 : BN) / 4;  // groups of four output columns per tile row
    constexpr int RPP = 256 / OC4;                               // rows per pass of the block
    const int oc = (threadIdx.x % OC4) * 4;                      // first output column of the thread inside the tile
    const int pc = EPI == EPI_SWIGLU ? (oc / 32) * 64 + oc % 32 : oc;  // its packed column inside the tile
    const int gp = t.nt * BN + pc;                               // packed column of the launch
    const int col = EPI == EPI_SWIGLU ? (gp / 64) * 32 + gp % 32 : gp;  // output column
    float4 sc0 = make_float4(1.f, 1.f, 1.f, 1.f), sc1 = sc0;
    if (FP8 && col < p.N) {
        sc0 = *(const float4*)(p.col_scale + (size_t)t.g * p.ncs + col);
        if constexpr (EPI == EPI_SWIGLU) sc1 = *(const float4*)(p.col_scale2 + (size_t)t.g * p.ncs + col);
    }
    bf16_t* C = (bf16_t*)p.C;
    const int r_end = min((slab + 1) * (BM / RSL), t.rv);
    for (int r = slab * (BM / RSL) + threadIdx.x / OC4; r < r_end; r += RPP) {
        const float* w = ws + (size_t)r * BN + gg_packed_row<FP8>(pc);  // (parts are stored by row of the weight tile)
        float4 a = *(const float4*)w, b = make_float4(0.f, 0.f, 0.f, 0.f);
        if constexpr (EPI == EPI_SWIGLU) b = *(const float4*)(w + 32);
        for (int part = 1; part < plan.P; ++part) {
            const float* wp = w + (size_t)part * (BM * BN);
            const float4 v = *(const float4*)wp;
            a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w;
            if constexpr (EPI == EPI_SWIGLU) {
                const float4 u = *(const float4*)(wp + 32);
                b.x += u.x; b.y += u.y; b.z += u.z; b.w += u.w;
            }
        }
        const size_t grow = (size_t)(t.row0 + r);
        float rs = 1.f;
        if constexpr (FP8 || EPI == EPI_GATE) rs = p.row_scale ? p.row_scale[grow] : 1.f;  // (fp8 down projection: a gate, or nothing)
        float av[4] = {a.x, a.y, a.z, a.w}, bv[4] = {b.x, b.y, b.z, b.w};
        if constexpr (!FP8 && EPI != EPI_NONE && EPI != EPI_GATE) {
            if (p.C2 && col < p.N) {  // the values before the activation, kept for the backward pass (rows are never remapped there)
                constexpr int W2 = EPI == EPI_SWIGLU ? 2 : 1;
                bf16_t* r2 = (bf16_t*)p.C2 + grow * (size_t)p.ldc * W2 + (EPI == EPI_SWIGLU ? gp : col);
                uint2 o2;
                o2.x = gg_pack_bf16(av[0], av[1]); o2.y = gg_pack_bf16(av[2], av[3]);
                *(uint2*)r2 = o2;
                if constexpr (EPI == EPI_SWIGLU) {
                    o2.x = gg_pack_bf16(bv[0], bv[1]); o2.y = gg_pack_bf16(bv[2], bv[3]);
                    *(uint2*)(r2 + 32) = o2;
                }
            }
        }
        const float c0[4] = {sc0.x, sc0.y, sc0.z, sc0.w}, c1[4] = {sc1.x, sc1.y, sc1.z, sc1.w};
        float x[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if constexpr (EPI == EPI_SWIGLU) {
                float gv = av[e], uv = bv[e];
                if constexpr (FP8) { gv *= c0[e] * rs; uv *= c1[e] * rs; }
                x[e] = act_silu_fast(gv) * uv;
            } else {
                float v = av[e];
                if constexpr (FP8) v *= c0[e] * rs;
                if constexpr (!FP8 && EPI == EPI_GATE) v *= rs;
                if constexpr (EPI == EPI_GELU) v = act_gelu(v);
                if constexpr (EPI == EPI_SILU) v = act_silu_fast(v);
                x[e] = v;
            }
        }
        const int crow = p.c_map ? p.c_map[grow] : 0;
        if constexpr (FP8 && EPI == EPI_SWIGLU) {
            // quantised output, as in the GEMM kernel's epilogue: the eight threads that hold a block of 32 columns of this
            // row (consecutive lanes; every thread of the block is in the loop together: r depends on threadIdx.x / OC4 only)
            float am = fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3])));
            if (col >= p.N) am = 0.f;
#pragma unroll
            for (int off = 1; off < 8; off <<= 1) am = fmaxf(am, __shfl_xor(am, off, WAVE));
            const int sbyte = gg_block_scale_byte(__float_as_uint(am));
            const float inv = __uint_as_float(gg_block_inv_bits(sbyte));
            int cd = 0;
            cd = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(x[0], inv), __fmul_rn(x[1], inv), cd, false);
            cd = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(x[2], inv), __fmul_rn(x[3], inv), cd, true);
            if (col < p.N && crow >= 0) {
                const size_t orow = p.c_map ? (size_t)crow : grow;
                *(uint32_t*)((uint8_t*)p.C + orow * p.ldc + col) = (uint32_t)cd;
                if ((col & 31) == 0) p.c_bscale[orow * p.bs_pitch + col / 32] = (uint8_t)sbyte;
            }
        } else if (col < p.N && crow >= 0) {
            uint2 o;
            o.x = gg_pack_bf16(x[0], x[1]);
            o.y = gg_pack_bf16(x[2], x[3]);
            *(uint2*)(C + (p.c_map ? (size_t)crow : grow) * p.ldc + col) = o;
        }
    }
}

// ---- one-time weight re-tiling: w [E_l,K,N] (N contiguous) -> out [E_l][K/SK][Npad][SK], SK = one LDS
// stage of K (ROWB bytes): the B tile of a stage is one contiguous 32 KB block -----------------------
// With w_up, gate and up columns are interleaved in groups of 32: packed col = (n/32)*64 + {0,32} + n%32.
template <typename T>
__global__ __launch_bounds__(256) void prepack_kernel(const T* __restrict__ w, const T* __restrict__ w_up, T* __restrict__ out,
                                                       int K, int N, int Npad) {
    __shared__ T tile[64][64 + 2];
    const int e = blockIdx.z;
    const int k0 = blockIdx.y * 64, n0 = blockIdx.x * 64;  // n0 in source columns
    const T* src = w + (size_t)e * K * N;
    const T* src2 = w_up ? w_up + (size_t)e * K * N : nullptr;
    T* dst = out + (size_t)e * Npad * K;
    constexpr int SK = ROWB / (int)sizeof(T);  // K elements per slab
    for (int pass = 0; pass < (src2 ? 2 : 1); ++pass) {
        const T* s = pass ? src2 : src;
        for (int i = threadIdx.x; i < 64 * 64; i += 256) {
            const int kk = i / 64, nn = i % 64;
            tile[kk][nn] = (k0 + kk < K && n0 + nn < N) ? s[(size_t)(k0 + kk) * N + n0 + nn] : (T)0;
        }
        __syncthreads();
        for (int i = threadIdx.x; i < 64 * 64; i += 256) {
            const int nn = i / 64, kk = i % 64;
            const int n = n0 + nn;
            // (columns [N, next multiple of 64) leave as the zeros they were loaded as: the rows of a group of 32 are
            // permuted, so a partly filled group cannot be zeroed as a range of rows)
            const int np = src2 ? ((n >> 5) * 64 + pass * 32 + (n & 31)) : n;
            if ((n < N || (!src2 && np < Npad)) && k0 + kk < K) {
                const int k = k0 + kk;
                dst[((size_t)(k / SK) * Npad + gg_packed_row<sizeof(T) == 1>(np)) * SK + (k % SK)] = tile[kk][nn];
            }
        }
        __syncthreads();
    }
}

template <typename T>
__global__ void zero_pad_rows_kernel(T* __restrict__ out, int K, int Nreal, int Npad) {
    // rows [Nreal, Npad) of every K slab of every expert's packed matrix (Nreal a multiple of 32: whole groups)
    constexpr int SK = ROWB / (int)sizeof(T);
    const int e = blockIdx.y;
    const size_t per_slab = (size_t)(Npad - Nreal) * SK;
    const size_t n = per_slab * (size_t)(K / SK);
    T* dst = out + (size_t)e * Npad * K;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const size_t slab = i / per_slab, r = i % per_slab;
        dst[(slab * Npad + Nreal) * SK + r] = (T)0;
    }
}

// ---- fp32 path: plain tiled FMA kernel, weights in the reference layout ------------------------------
// C[rows of g] = epi(A[rows of g] @ W[g] (, A @ Wup[g])); 64x64 tiles, 16x16 threads, 4x4 per thread; K in slabs
// of 64 through LDS, the next slab fetched into registers while the current one is multiplied (the workloads of
// this path are small: what counts is that no memory latency is left exposed per slab).
template <int EPI>
__global__ __launch_bounds__(256) void grouped_gemm_f32_kernel(const float* __restrict__ A, const float* __restrict__ Wt,
                                                                const float* __restrict__ Wup, float* __restrict__ C,
                                                                const int32_t* __restrict__ cnt, int E_l, int K, int N,
                                                                int S_rows) {
    constexpr int KC = 64;                       // K per slab
    constexpr int PT = 64 * KC / 256;            // elements of each operand per thread and slab
    __shared__ float As[KC][64 + 4];
    __shared__ float Bs[KC][64];
    __shared__ float Us[EPI == EPI_SWIGLU ? KC : 1][64];
    __shared__ int s_g, s_row0, s_rv;
    if (threadIdx.x == 0) {
        int mt = blockIdx.y, rs = 0, g = 0, found = 0;
        for (; g < E_l; ++g) {
            const int c = max(cnt[g], 0);
            const int t = (c + 63) / 64;
            if (mt < t) { found = 1; s_row0 = rs + mt * 64; s_rv = min(min(64, c - mt * 64), S_rows - (rs + mt * 64)); break; }
            mt -= t;
            rs += c;
        }
        s_g = found ? g : -1;
    }
    __syncthreads();
    const int g = s_g;
    if (g < 0 || s_rv <= 0) return;
    const int row0 = s_row0, rv = s_rv, n0 = blockIdx.x * 64;
    const float* W = Wt + (size_t)g * K * N;
    const float* U = EPI == EPI_SWIGLU ? Wup + (size_t)g * K * N : nullptr;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    float acc[4][4] = {}, acu[4][4] = {};
    float ra[PT], rb[PT], ru[EPI == EPI_SWIGLU ? PT : 1];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int q = 0; q < PT; ++q) {
            const int i = threadIdx.x + q * 256;
            const int r = i / KC, kk = i % KC;          // A: consecutive threads walk K
            ra[q] = (r < rv && k0 + kk < K) ? A[(size_t)(row0 + r) * K + k0 + kk] : 0.f;
            const int kb = i / 64, nn = i % 64;          // W: consecutive threads walk N
            const bool ok = k0 + kb < K && n0 + nn < N;
            rb[q] = ok ? W[(size_t)(k0 + kb) * N + n0 + nn] : 0.f;
            if constexpr (EPI == EPI_SWIGLU) ru[q] = ok ? U[(size_t)(k0 + kb) * N + n0 + nn] : 0.f;
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += KC) {
#pragma unroll
        for (int q = 0; q < PT; ++q) {
            const int i = threadIdx.x + q * 256;
            As[i % KC][i / KC] = ra[q];
            Bs[i / 64][i % 64] = rb[q];
            if constexpr (EPI == EPI_SWIGLU) Us[i / 64][i % 64] = ru[q];
        }
        __syncthreads();
        if (k0 + KC < K) fetch(k0 + KC);
        // slab positions past K hold zeros: adding +0 products leaves every sum as it is
#pragma unroll 8
        for (int kk = 0; kk < KC; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
            if constexpr (EPI == EPI_SWIGLU) {
                float u[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) u[j] = Us[kk][tx * 4 + j];
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acu[i][j] = fmaf(a[i], u[j], acu[i][j]);
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = ty * 4 + i;
        if (r >= rv) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = n0 + tx * 4 + j;
            if (c >= N) continue;
            float x = acc[i][j];
            if constexpr (EPI == EPI_GELU) x = act_gelu(x);
            if constexpr (EPI == EPI_SILU) x = act_silu(x);
            if constexpr (EPI == EPI_SWIGLU) x = act_silu(x) * acu[i][j];
            C[(size_t)(row0 + r) * N + c] = x;
        }
    }
}

// ---- per-row fp8 quantisation of bf16 rows (one wave per row) -------------------------------------
// Rows of up to 64 * NV * 8 columns are held in registers between the amax pass and the conversion, so
// they are read from memory once; longer rows are read twice.
__device__ __forceinline__ float fp8_row_amax(const uint4& v, float amax) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        amax = fmaxf(amax, fabsf(__uint_as_float(w[i] << 16)));
        amax = fmaxf(amax, fabsf(__uint_as_float(w[i] & 0xffff0000u)));
    }
    return amax;
}
__device__ __forceinline__ uint2 fp8_row_convert(const uint4& v, float inv) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    float f[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = __fmul_rn(__uint_as_float(w[i] << 16), inv);
        f[2 * i + 1] = __fmul_rn(__uint_as_float(w[i] & 0xffff0000u), inv);
    }
    int lo = 0, hi = 0;
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], lo, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], hi, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
    return make_uint2((uint32_t)lo, (uint32_t)hi);
}

template <int NV>  // 16-byte vectors per lane kept in registers (0: stream the row twice)
__global__ __launch_bounds__(256) void quantize_rows_fp8_kernel(const bf16_t* __restrict__ x, int rows, int cols,
                                                                 uint8_t* __restrict__ q, float* __restrict__ scale,
                                                                 const int32_t* __restrict__ n_rows_dev,
                                                                 const int32_t* __restrict__ src_map) {
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int limit = n_rows_dev ? min(rows, *n_rows_dev) : rows;
    const int nv = cols / 8;
    for (int r = blockIdx.x * 4 + wave; r < limit; r += gridDim.x * 4) {
        const uint4* src = (const uint4*)(x + (size_t)(src_map ? max(src_map[r], 0) : r) * cols);
        uint4 held[NV > 0 ? NV : 1];
        float amax = 0.f;
        if constexpr (NV > 0) {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int c = lane + i * WAVE;
                held[i] = c < nv ? src[c] : make_uint4(0, 0, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < NV; ++i) amax = fp8_row_amax(held[i], amax);
        } else {
            for (int c = lane; c < nv; c += WAVE) amax = fp8_row_amax(src[c], amax);
        }
#pragma unroll
        for (int off = WAVE / 2; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, WAVE));
        const bool zero = amax == 0.f;
        const float inv = zero ? 1.f : __fdiv_rn(448.f, amax);
        if (lane == 0) scale[r] = zero ? 1.f : __fdiv_rn(amax, 448.f);
        uint2* dst = (uint2*)(q + (size_t)r * cols);
        if constexpr (NV > 0) {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int c = lane + i * WAVE;
                if (c < nv) dst[c] = fp8_row_convert(held[i], inv);
            }
        } else {
            for (int c = lane; c < nv; c += WAVE) dst[c] = fp8_row_convert(src[c], inv);
        }
    }
}

// ---- quantise and pack in one pass: the token rows leave the source as fp8 codes and one scale per row -----------------
// Per-row quantisation commutes with moving rows: send_q / send_scale hold, slot for slot, what quantize_rows_fp8 would make
// of the bf16 send buffer (padding slots: codes 0, scale 1, as for an all-zero row) -- so the destination can feed them to
// the fp8 GEMM as they arrive, and half the bytes cross.  Units [0, T) of the launch are tokens (one wave each: the row is
// read once, quantised in registers, stored to its k slots); the units after them are runs of PACKQ_ZR slots that are
// written only where they are padding.
constexpr int PACKQ_ZR = 8;
template <int NV>
__global__ __launch_bounds__(256) void pack_tokens_fp8_kernel(const bf16_t* __restrict__ x, int T, int cols,
                                                               const int32_t* __restrict__ idx, const int32_t* __restrict__ pos,
                                                               const int32_t* __restrict__ dst_sizes,
                                                               const int32_t* __restrict__ dst_offsets, int k, int E_l, int W, int M,
                                                               uint8_t* __restrict__ send_q, float* __restrict__ send_scale,
                                                               int32_t* __restrict__ status, const float* __restrict__ gate,
                                                               float* __restrict__ send_gate) {
    // (gate / send_gate, both or neither: the slot's top-k gate travels with its row, zero in the padding slots)
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const int nv = cols / 8;  // 16-byte vectors of bf16 per row = 8-byte vectors of codes
    const int n_slots = W * M;
    const int n_units = T + (n_slots + PACKQ_ZR - 1) / PACKQ_ZR;
    for (int r = blockIdx.x * 4 + wave; r < n_units; r += gridDim.x * 4) {
        if (r >= T) {
            const int s0 = (r - T) * PACKQ_ZR, s1 = min(s0 + PACKQ_ZR, n_slots);
            int d = s0 / M, m = s0 % M;
            int cnt = dst_sizes[d];
            for (int sl = s0; sl < s1; ++sl) {
                if (m == 0 && cnt > M && status && lane == 0) *status = 1;
                if (m >= cnt) {
                    uint2* o = (uint2*)(send_q + (size_t)sl * cols);
                    for (int c = lane; c < nv; c += WAVE) o[c] = make_uint2(0u, 0u);
                    if (lane == 0) send_scale[sl] = 1.f;
                    if (send_gate && lane == 0) send_gate[sl] = 0.f;
                }
                if (++m == M && sl + 1 < s1) { m = 0; cnt = dst_sizes[++d]; }
            }
            continue;
        }
        int drow[MOE_MAX_TOPK];
#pragma unroll
        for (int j = 0; j < MOE_MAX_TOPK; ++j) {
            drow[j] = -1;
            if (j < k) {
                const int d = idx[(size_t)r * k + j] / E_l;
                const bool d_ok = (unsigned)d < (unsigned)W;
                const int m = pos[(size_t)r * k + j] - dst_offsets[d_ok ? d : 0];
                if (d_ok && (unsigned)m < (unsigned)M) drow[j] = d * M + m;
                if (send_gate && drow[j] >= 0 && lane == 0) send_gate[drow[j]] = gate[(size_t)r * k + j];
            }
        }
        const uint4* src = (const uint4*)(x + (size_t)r * cols);
        uint4 held[NV > 0 ? NV : 1];
        float amax = 0.f;
        if constexpr (NV > 0) {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int c = lane + i * WAVE;
                held[i] = c < nv ? src[c] : make_uint4(0, 0, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < NV; ++i) amax = fp8_row_amax(held[i], amax);
        } else {
            for (int c = lane; c < nv; c += WAVE) amax = fp8_row_amax(src[c], amax);
        }
#pragma unroll
        for (int off = WAVE / 2; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, WAVE));
        const bool zero = amax == 0.f;
        const float inv = zero ? 1.f : __fdiv_rn(448.f, amax);
        const float sc = zero ? 1.f : __fdiv_rn(amax, 448.f);
        if constexpr (NV > 0) {
            uint2 code[NV];
#pragma unroll
            for (int i = 0; i < NV; ++i) code[i] = fp8_row_convert(held[i], inv);
#pragma unroll
            for (int j = 0; j < MOE_MAX_TOPK; ++j) {
                if (j < k && drow[j] >= 0) {
                    uint2* o = (uint2*)(send_q + (size_t)drow[j] * cols);
#pragma unroll
                    for (int i = 0; i < NV; ++i) {
                        const int c = lane + i * WAVE;
                        if (c < nv) o[c] = code[i];
                    }
                    if (lane == 0) send_scale[drow[j]] = sc;
                }
            }
        } else {
            for (int c = lane; c < nv; c += WAVE) {
                const uint2 code = fp8_row_convert(src[c], inv);
#pragma unroll
                for (int j = 0; j < MOE_MAX_TOPK; ++j)
                    if (j < k && drow[j] >= 0) ((uint2*)(send_q + (size_t)drow[j] * cols))[c] = code;
            }
#pragma unroll
            for (int j = 0; j < MOE_MAX_TOPK; ++j)
                if (j < k && drow[j] >= 0 && lane == 0) send_scale[drow[j]] = sc;
        }
    }
}

// out[r] = scale[map[r]] (map NULL: scale[r]; a negative entry takes row 0, like the GEMM's row gather)
__global__ __launch_bounds__(256) void gather_scale_kernel(const float* __restrict__ scale, const int32_t* __restrict__ map, int n,
                                                            float* __restrict__ out) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r < n) out[r] = scale[map ? max(map[r], 0) : r];
}

// ---- backward pass helpers -----------------------------------------------------------------------------------------
// Re-tiling of w [E_l,K,N] as the weights of the TRANSPOSED product (d tokens = d out @ w^T: reduction over N, K output
// columns): out[e][n / SK][k][n % SK] = w[e][k][n], rows k in [K, Kpad) zero.  No transposition is involved: the 64-byte
// runs of n are contiguous on both sides.  With w_up the slabs alternate (32 n of w, 32 n of w_up, ...), which is the
// column order of the fused gate/up product, so the same call serves d tokens = [d gate | d up] @ [w_gate | w_up]^T.
template <typename T>
__global__ __launch_bounds__(256) void prepack_t_kernel(const T* __restrict__ w, const T* __restrict__ w_up, T* __restrict__ out,
                                                         int K, int N, int Kpad) {
    constexpr int SK = ROWB / (int)sizeof(T);
    constexpr int VPS = ROWB / 16;  // 16-byte vectors per 64-byte run
    const int e = blockIdx.y;
    const int nsl = N / SK, passes = w_up ? 2 : 1;
    const size_t total = (size_t)nsl * passes * Kpad * VPS;
    const uint4 z = make_uint4(0, 0, 0, 0);
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const int v = (int)(i % VPS);
        const int k = (int)((i / VPS) % Kpad);
        const int slab = (int)(i / ((size_t)VPS * Kpad));  // output slab: (n / SK) * passes + pass
        const int ns = slab / passes, pass = slab % passes;
        const T* src = (pass ? w_up : w) + (size_t)e * K * N;
        uint4 val = z;
        const int kc = gg_packed_col<sizeof(T) == 1>(k);  // the output column of the transposed product this row stands for
        if (kc < K) val = *reinterpret_cast<const uint4*>(src + (size_t)kc * N + (size_t)ns * SK + v * (16 / (int)sizeof(T)));
        *reinterpret_cast<uint4*>(out + (((size_t)e * nsl * passes + slab) * Kpad + k) * SK + v * (16 / (int)sizeof(T))) = val;
    }
}

// Operands of the weight-gradient product d w[g] = x_g^T @ dy_g, whose reduction runs over the rows of group g: both
// matrices are needed with the row index fastest.  Rows are renumbered s -> s' so that every group starts at a
// multiple of 64 (two K stages of the GEMM) and its tail up to the next multiple of 64 is zero.  A block moves 64 rows
// (one group's, never two) x 64 columns through LDS.
//   SLAB = false: out = x^T, [cols, ld_out] row-major                       (the GEMM's activation operand)
//   SLAB = true : out = the weight layout over the padded rows, [ld_out / SK][Npad][SK]  (the GEMM's weight operand)
//                with split_F > 0 the input columns are in the fused gate/up order (32 gate, 32 up, ...) and leave in
//                the order [all gate | all up], so that the product's columns are the two weight gradients side by side
template <bool SLAB>
__global__ __launch_bounds__(256) void dw_operand_kernel(const uint16_t* __restrict__ in, const int32_t* __restrict__ cnt, int E_l,
                                                          int S_rows, int cols, uint16_t* __restrict__ out, int ld_out, int Npad,
                                                          int split_F) {
    __shared__ uint16_t tile[64][64 + 2];
    __shared__ int s_src0, s_valid;
    if (threadIdx.x == 0) {
        // padded block blockIdx.y -> (first source row, valid rows); blocks past the padded total have nothing to do
        int pb = 0, rs = 0, src0 = -1, valid = 0;
        for (int g = 0; g < E_l; ++g) {
            const int c = min(max(cnt[g], 0), max(S_rows - rs, 0));
            const int nb = (c + 63) / 64;
            if ((int)blockIdx.y < pb + nb) {
                const int j = blockIdx.y - pb;
                src0 = rs + j * 64;
                valid = min(64, c - j * 64);
                break;
            }
            pb += nb;
            rs += c;
        }
        s_src0 = src0;
        s_valid = valid;
    }
    __syncthreads();
    const int src0 = s_src0, valid = s_valid;
    if (src0 < 0) return;
    const int c0 = blockIdx.x * 64;
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int r = i / 64, c = i % 64;
        tile[r][c] = (r < valid && c0 + c < cols) ? in[(size_t)(src0 + r) * cols + c0 + c] : (uint16_t)0;
    }
    __syncthreads();
    const int sp0 = blockIdx.y * 64;  // first padded row of the block
    constexpr int SK = ROWB / 2;
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int c = i / 64, r = i % 64;  // consecutive threads walk the rows: contiguous in both output layouts
        if (c0 + c >= (SLAB ? Npad : cols)) continue;
        const uint16_t v = tile[r][c];  // (columns in [cols, Npad) were loaded as zeros)
        const int sp = sp0 + r;
        if constexpr (SLAB) {
            int oc = c0 + c;
            if (split_F > 0 && oc < 2 * split_F) oc = ((oc % 64) / 32) * split_F + (oc / 64) * 32 + oc % 32;
            out[((size_t)(sp / SK) * Npad + gg_packed_row<false>(oc)) * SK + sp % SK] = v;
        } else {
            out[(size_t)(c0 + c) * ld_out + sp] = v;
        }
    }
}

// d w[g] <- 0 for the groups that received no row (the GEMM has no tile for them)
__global__ __launch_bounds__(256) void dw_zero_empty_kernel(uint4* __restrict__ dw, const int32_t* __restrict__ cnt,
                                                             size_t vec_per_group, int src_rows) {
    // (a group whose rows all lie past the end of the operands counts as empty, as in the GEMM's own tables)
    int before = 0;
    for (int e = 0; e < (int)blockIdx.y; ++e) before += max(cnt[e], 0);
    if (min(max(cnt[blockIdx.y], 0), max(src_rows - before, 0)) > 0) return;
    uint4* d = dw + (size_t)blockIdx.y * vec_per_group;
    const uint4 z = make_uint4(0, 0, 0, 0);
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < vec_per_group; i += (size_t)gridDim.x * blockDim.x) d[i] = z;
}

// Gradient through the activation of the expert MLP.  a1: the pre-activations as the first GEMM produces them without an
// epilogue ([rows, F] for GELU / SiLU; [rows, 2F] in the fused gate/up column order -- 32 gate columns, their 32 up
// columns, ... -- for SwiGLU); dh: gradient of the hidden activation [rows, F]; out: gradient of a1, same layout as a1.
//   GELU (erf):  dx = dh * (Phi(x) + x phi(x));   SiLU: dx = dh * s (1 + x (1 - s)), s = sigmoid(x);
//   SwiGLU h = silu(g) u:  dg = dh * u * silu'(g),  du = dh * silu(g).
template <typename T>
__device__ __forceinline__ void store_f32(T* p, float v);
template <>
__device__ __forceinline__ void store_f32<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void store_f32<bf16_t>(bf16_t* p, float v) { *p = f32_to_bf16(v); }

template <int EPI, typename T>
__global__ __launch_bounds__(256) void act_backward_kernel(const T* __restrict__ a1, const T* __restrict__ dh,
                                                            T* __restrict__ out, size_t rows, int F) {
    const size_t total = rows * (size_t)F;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / F;
        const int n = (int)(i % F);
        const float d = load_f32<T>(dh + i);
        if constexpr (EPI == EPI_SWIGLU) {
            const size_t base = r * (size_t)(2 * F) + (size_t)(n / 32) * 64 + n % 32;
            const float gv = load_f32<T>(a1 + base), uv = load_f32<T>(a1 + base + 32);
            const float s = 1.0f / (1.0f + __expf(-gv));
            store_f32<T>(out + base, d * uv * (s * (1.0f + gv * (1.0f - s))));
            store_f32<T>(out + base + 32, d * (gv * s));
        } else {
            const float x = load_f32<T>(a1 + i);
            float dv = d;
            if constexpr (EPI == EPI_GELU)
                dv = d * (0.5f * (1.0f + erff(x * 0.70710678118654752440f)) + x * 0.39894228040143267794f * __expf(-0.5f * x * x));
            if constexpr (EPI == EPI_SILU) {
                const float s = 1.0f / (1.0f + __expf(-x));
                dv = d * (s * (1.0f + x * (1.0f - s)));
            }
            store_f32<T>(out + i, dv);
        }
    }
}

// fp32 path of the backward pass (plumbing-size workloads): d w[g] = x_g^T @ dy_g, 64 x 64 output tiles, the group's
// rows in slabs of 32 through LDS; and the plain transposition w [E,K,N] -> [E,N,K] that d tokens = dy @ w^T needs.
__global__ __launch_bounds__(256) void grouped_dw_f32_kernel(const float* __restrict__ x, const float* __restrict__ dy,
                                                              const int32_t* __restrict__ cnt, int E_l, int K, int N, int S_rows,
                                                              float* __restrict__ dw) {
    constexpr int SC = 32;
    __shared__ float xs[SC][64 + 1];
    __shared__ float ys[SC][64 + 1];
    const int g = blockIdx.z, k0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
    int row0 = 0;
    for (int e = 0; e < g; ++e) row0 += max(cnt[e], 0);
    const int c = min(max(cnt[g], 0), max(S_rows - row0, 0));
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    float acc[4][4] = {};
    for (int s0 = 0; s0 < c; s0 += SC) {
        for (int i = threadIdx.x; i < SC * 64; i += 256) {
            const int r = i / 64, cc = i % 64;
            const bool live = s0 + r < c;
            xs[r][cc] = (live && k0 + cc < K) ? x[(size_t)(row0 + s0 + r) * K + k0 + cc] : 0.f;
            ys[r][cc] = (live && n0 + cc < N) ? dy[(size_t)(row0 + s0 + r) * N + n0 + cc] : 0.f;
        }
        __syncthreads();
#pragma unroll 4
        for (int r = 0; r < SC; ++r) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[r][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ys[r][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + ty * 4 + i, n = n0 + tx * 4 + j;
            if (k < K && n < N) dw[((size_t)g * K + k) * N + n] = acc[i][j];
        }
}

__global__ __launch_bounds__(256) void transpose_f32_kernel(const float* __restrict__ w, float* __restrict__ out, int K, int N) {
    __shared__ float tile[32][33];
    const float* src = w + (size_t)blockIdx.z * K * N;
    float* dst = out + (size_t)blockIdx.z * K * N;
    const int k0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
    for (int i = threadIdx.x; i < 1024; i += 256) {
        const int k = i / 32, n = i % 32;
        tile[k][n] = (k0 + k < K && n0 + n < N) ? src[(size_t)(k0 + k) * N + n0 + n] : 0.f;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 1024; i += 256) {
        const int n = i / 32, k = i % 32;
        if (k0 + k < K && n0 + n < N) dst[(size_t)(n0 + n) * K + k0 + k] = tile[k][n];
    }
}

int num_cus() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) cus = prop.multiProcessorCount;
        if (cus <= 0) cus = 256;
    }
    return cus;
}

int round_up(int a, int b) { return (a + b - 1) / b * b; }

// moe_diag_gemm_trace: where the next forward GEMM launches of this process leave time stamps (not thread-safe: a diagnostic)
struct { unsigned long long* buf; int flags; } g_trace = {nullptr, 0};

template <bool FP8>
int launch_gemm(const GemmParams& p_in, int epi, hipStream_t s, void* part_ws = nullptr, size_t part_ws_bytes = 0) {
    const int grid = num_cus();
    GemmParams p = p_in;
    const bool traced = g_trace.buf && (!(g_trace.flags & 0x300) || (g_trace.flags & (epi == EPI_NONE ? 0x100 : 0x200)));
    if (traced) {  // (see moe_diag_gemm_trace: whole tiles only, so that every tile leaves its stamps)
        p.trace = g_trace.buf;
        p.trace_flags = g_trace.flags;
        part_ws = nullptr;
    }
    // 256-row or 128-row tiles: the host knows only the total row count, so it compares the estimated number
    // of rounds of the persistent grid (every group adds about half a tile of ragged tail); a 128-row tile
    // costs about 0.62 of a 256-row one
    const int nt = p.Npad / GG_BN;
    const double t256 = ((double)p.S_rows / 256 + 0.5 * p.E_l) * nt, t128 = ((double)p.S_rows / 128 + 0.5 * p.E_l) * nt;
    const bool small_m = 0.62 * ceil(t128 / grid) < ceil(t256 / grid);
    // with a workspace, the tiles of a last round that fills at most a quarter of the grid are split along K
    // (decided on the device from the row counts); the reduction kernel finds nothing to do otherwise
    p.part_ws = nullptr;
    p.max_units = 0;
    if (part_ws) {
        p.max_units = (int)std::min<size_t>(part_ws_bytes / ((size_t)(small_m ? 128 : 256) * GG_BN * sizeof(float)), (size_t)grid);
        if (p.max_units >= 2) p.part_ws = (float*)part_ws;
    }
    const int red_blocks = (grid / 4) * GG_RED_SLABS;
    // A launch so small that all its tiles are certain to be split (whatever the row counts turn out to be, there are at most
    // ub of them: every group adds at most one partly filled row of tiles) has no whole tile: the first kernel is left out.
    // gg_plan finds two parts or more whenever 4 tail <= grid, the K range has 16 stages and the workspace holds 2 tail units.
    const int bm = small_m ? 128 : 256, nk = p.K * (FP8 ? 1 : 2) / ROWB;
    const long long ub = ((long long)(p.S_rows + bm - 1) / bm + p.E_l) * nt;
    const bool all_split = p.part_ws && red_blocks > 0 && 4 * ub <= grid && nk >= 2 * GG_MIN_PART_STAGES && p.max_units >= 2 * ub;
    // fp8 without activation is the down projection of the expert MLP: its activation operand is block-scaled
#define GG_LAUNCH(BMv, NWMv, EPIv)                                                                        \
    do {                                                                                                  \
        constexpr bool BSAv = FP8 && EPIv == EPI_NONE;                                                    \
        if (traced) {                                                                                     \
            if constexpr (BMv == 256 && (EPIv == EPI_NONE || EPIv == EPI_SWIGLU))                         \
                grouped_gemm_kernel<BMv, NWMv, EPIv, FP8, false, false, BSAv, true><<<grid, NWMv * 2 * WAVE, 0, s>>>(p); \
            else return moe_fail(MOE_ERR_UNSUPPORTED, "grouped_gemm: no time-stamping instantiation for this launch (256-row tiles, no activation or SwiGLU)"); \
            break;                                                                                        \
        }                                                                                                 \
        if (!all_split) grouped_gemm_kernel<BMv, NWMv, EPIv, FP8, false, false, BSAv><<<grid, NWMv * 2 * WAVE, 0, s>>>(p); \
        if (p.part_ws && red_blocks > 0) {                                                                \
            /* (the launch that takes parts stores raw partial sums: one instantiation whatever the epilogue) */ \
            grouped_gemm_kernel<BMv, NWMv, EPI_NONE, FP8, true, false, BSAv><<<grid, NWMv * 2 * WAVE, 0, s>>>(p); \
            gg_reduce_parts_kernel<BMv, EPIv, FP8><<<red_blocks, 256, 0, s>>>(p, grid);                    \
        }                                                                                                 \
    } while (0)
#define GG_EPI(EPIv)                          \
    do {                                      \
        if (small_m) GG_LAUNCH(128, 2, EPIv); \
        else GG_LAUNCH(256, (FP8 ? (EPIv == EPI_NONE ? GG_FP8_BSA_NWM : GG_FP8_NWM) : GG_BIG_NWM), EPIv); \
    } while (0)
    switch (epi) {
        case EPI_NONE:
            if (FP8 && !p.a_bscale) return moe_fail(MOE_ERR_INVALID, "grouped_gemm: the fp8 down projection needs block scales");
            GG_EPI(EPI_NONE);
            break;
        // (no fp8 entry point asks for these two: not instantiated)
        case EPI_GELU: if constexpr (FP8) return moe_fail(MOE_ERR_UNSUPPORTED, "grouped_gemm: fp8 with activation %d", epi); else GG_EPI(EPI_GELU); break;
        case EPI_SILU: if constexpr (FP8) return moe_fail(MOE_ERR_UNSUPPORTED, "grouped_gemm: fp8 with activation %d", epi); else GG_EPI(EPI_SILU); break;
        case EPI_SWIGLU: GG_EPI(EPI_SWIGLU); break;
        case EPI_GATE: if constexpr (FP8) return moe_fail(MOE_ERR_UNSUPPORTED, "grouped_gemm: fp8 folds a gate into its row scale"); else GG_EPI(EPI_GATE); break;
        default: return moe_fail(MOE_ERR_INVALID, "grouped_gemm: activation %d", epi);
    }
#undef GG_EPI
#undef GG_LAUNCH
    return moe_check_launch("grouped_gemm");
}

int launch_f32(const float* A, const float* W, const float* U, float* C, const int32_t* cnt, int E_l, int K, int N, int S_rows,
               int epi, hipStream_t s) {
    if (S_rows == 0) return MOE_OK;
    dim3 grid(ceil_div(N, 64), ceil_div(S_rows, 64) + E_l);
    switch (epi) {
        case EPI_NONE: grouped_gemm_f32_kernel<EPI_NONE><<<grid, 256, 0, s>>>(A, W, U, C, cnt, E_l, K, N, S_rows); break;
        case EPI_GELU: grouped_gemm_f32_kernel<EPI_GELU><<<grid, 256, 0, s>>>(A, W, U, C, cnt, E_l, K, N, S_rows); break;
        case EPI_SILU: grouped_gemm_f32_kernel<EPI_SILU><<<grid, 256, 0, s>>>(A, W, U, C, cnt, E_l, K, N, S_rows); break;
        case EPI_SWIGLU: grouped_gemm_f32_kernel<EPI_SWIGLU><<<grid, 256, 0, s>>>(A, W, U, C, cnt, E_l, K, N, S_rows); break;
        default: return moe_fail(MOE_ERR_INVALID, "grouped_gemm: activation %d", epi);
    }
    return moe_check_launch("grouped_gemm_f32");
}

template <typename T>
int launch_prepack(const T* w, const T* w_up, int E_l, int K, int N, T* out, hipStream_t s) {
    const int n_eff = N * (w_up ? 2 : 1);
    const int Npad = round_up(n_eff, GG_BN);
    const int n_zero = w_up ? n_eff : std::min(round_up(N, 64), Npad);  // (the re-tiling kernel writes the zeros up to there)
    if (Npad > n_zero) zero_pad_rows_kernel<T><<<dim3(64, E_l), 256, 0, s>>>(out, K, n_zero, Npad);
    prepack_kernel<T><<<dim3(ceil_div(N, 64), ceil_div(K, 64), E_l), 256, 0, s>>>(w, w_up, out, K, N, Npad);
    return moe_check_launch("prepack_weights");
}

}  // namespace moe_gg
using namespace moe_gg;

extern "C" size_t moe_diag_gemm_trace_words(void) { return (size_t)num_cus() * GG_TRACE_TILE_WORDS + GG_TRACE_BLOCK_WORDS; }

extern "C" int moe_diag_gemm_trace(unsigned long long* trace, size_t words, int flags) {
    MOE_REQUIRE(!trace || words >= moe_diag_gemm_trace_words(), MOE_ERR_WORKSPACE, "diag_gemm_trace: %zu words, %zu needed", words,
                moe_diag_gemm_trace_words());
    g_trace.buf = trace;
    g_trace.flags = trace ? flags : 0;
    return MOE_OK;
}

extern "C" size_t moe_prepack_bytes(int dtype, int E_l, int K, int N) {
    if (dtype == MOE_F32) return 0;
    const size_t es = dtype == MOE_BF16 ? 2 : 1;
    return (size_t)E_l * (size_t)round_up(N, GG_BN) * (size_t)K * es;
}

extern "C" int moe_prepack_weights(const void* w, const void* w_up, int dtype, int E_l, int K, int N, void* packed,
                                   moe_stream_t stream) {
    MOE_REQUIRE(dtype == MOE_BF16, MOE_ERR_INVALID, "prepack_weights: bf16 only (dtype %d)", dtype);
    MOE_REQUIRE(E_l > 0 && K > 0 && N > 0 && w && packed, MOE_ERR_INVALID, "prepack_weights: bad arguments");
    MOE_REQUIRE(!w_up || N % 32 == 0, MOE_ERR_UNSUPPORTED, "prepack_weights: gate/up interleave needs N %% 32 == 0 (N=%d)", N);
    return launch_prepack<uint16_t>((const uint16_t*)w, (const uint16_t*)w_up, E_l, K, N, (uint16_t*)packed, (hipStream_t)stream);
}

extern "C" int moe_prepack_weights_fp8(const uint8_t* w, const uint8_t* w_up, int E_l, int K, int N, uint8_t* packed,
                                       moe_stream_t stream) {
    MOE_REQUIRE(E_l > 0 && K > 0 && N > 0 && w && packed, MOE_ERR_INVALID, "prepack_weights_fp8: bad arguments");
    MOE_REQUIRE(!w_up || N % 32 == 0, MOE_ERR_UNSUPPORTED, "prepack_weights_fp8: gate/up interleave needs N %% 32 == 0");
    return launch_prepack<uint8_t>(w, w_up, E_l, K, N, packed, (hipStream_t)stream);
}

extern "C" int moe_grouped_gemm(const void* tokens, const void* weights, const int32_t* expert_cnt, int dtype, int S_rows,
                                int K, int N, int E_l, void* out, void* ws, size_t ws_bytes, moe_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    MOE_REQUIRE(S_rows >= 0 && K > 0 && N > 0 && E_l > 0 && E_l <= GG_MAXG, MOE_ERR_INVALID, "grouped_gemm: bad shape");
    if (S_rows == 0) return MOE_OK;
    MOE_REQUIRE(tokens && weights && expert_cnt && out, MOE_ERR_INVALID, "grouped_gemm: null pointer");
    if (dtype == MOE_F32)
        return launch_f32((const float*)tokens, (const float*)weights, nullptr, (float*)out, expert_cnt, E_l, K, N, S_rows,
                          EPI_NONE, s);
    MOE_REQUIRE(dtype == MOE_BF16, MOE_ERR_INVALID, "grouped_gemm: dtype %d", dtype);
    MOE_REQUIRE(K % 64 == 0 && N % 8 == 0, MOE_ERR_UNSUPPORTED, "grouped_gemm: bf16 needs K %% 64 == 0 and N %% 8 == 0 (K=%d N=%d)", K, N);
    MOE_REQUIRE(ws && ws_bytes >= moe_prepack_bytes(dtype, E_l, K, N), MOE_ERR_WORKSPACE, "grouped_gemm: workspace too small");
    int rc = launch_prepack<uint16_t>((const uint16_t*)weights, nullptr, E_l, K, N, (uint16_t*)ws, s);
    if (rc) return rc;
    GemmParams p{};
    p.A = (const uint8_t*)tokens; p.B = (const uint8_t*)ws; p.C = out; p.cnt = expert_cnt;
    p.E_l = E_l; p.K = K; p.N = N; p.Npad = round_up(N, GG_BN); p.ldc = N; p.S_rows = S_rows;
    return launch_gemm<false>(p, EPI_NONE, s);
}

extern "C" int moe_grouped_gemm_packed(const void* tokens, const void* packed, const int32_t* expert_cnt, int S_rows, int K,
                                       int N, int E_l, int act, void* out, moe_stream_t stream) {
    MOE_REQUIRE(S_rows >= 0 && K > 0 && N > 0 && E_l > 0 && E_l <= GG_MAXG, MOE_ERR_INVALID, "grouped_gemm_packed: bad shape");
    MOE_REQUIRE(act >= EPI_NONE && act <= EPI_SWIGLU, MOE_ERR_INVALID, "grouped_gemm_packed: activation %d", act);
    MOE_REQUIRE(K % 64 == 0 && N % 8 == 0, MOE_ERR_UNSUPPORTED, "grouped_gemm_packed: needs K %% 64 == 0 and N %% 8 == 0 (K=%d N=%d)", K, N);
    if (S_rows == 0) return MOE_OK;
    MOE_REQUIRE(tokens && packed && expert_cnt && out, MOE_ERR_INVALID, "grouped_gemm_packed: null pointer");
    GemmParams p{};
    p.A = (const uint8_t*)tokens; p.B = (const uint8_t*)packed; p.C = out; p.cnt = expert_cnt;
    p.E_l = E_l; p.K = K; p.N = N; p.ldc = N; p.S_rows = S_rows;
    p.Npad = round_up(act == EPI_SWIGLU ? 2 * N : N, GG_BN);
    return launch_gemm<false>(p, act, (hipStream_t)stream);
}

// The tile walk of a launch as the kernels compute it (host side of the same function; no GPU needed):
// out = {full, P, stages per part, work units}.  For callers that size workspaces and for tests.
extern "C" int moe_gemm_split_plan(int total_tiles, int grid, int k_stages, int max_units, int32_t* out) {
    MOE_REQUIRE(total_tiles >= 0 && grid > 0 && k_stages >= 2 && k_stages % 2 == 0 && max_units >= 0 && out, MOE_ERR_INVALID,
                "gemm_split_plan: bad arguments");
    const GgPlan pl = gg_plan(total_tiles, grid, k_stages, max_units >= 2, max_units);
    out[0] = pl.full; out[1] = pl.P; out[2] = pl.nkp; out[3] = pl.units;
    return MOE_OK;
}

extern "C" size_t moe_gemm_part_workspace_bytes(void) { return (size_t)num_cus() * 256 * GG_BN * sizeof(float); }

extern "C" int moe_grouped_gemm_mapped(const void* a_base, int a_rows, const int32_t* a_row_map, const void* packed,
                                       const int32_t* expert_cnt, int S_rows, int K, int N, int E_l, int act, void* out,
                                       int out_rows, const int32_t* c_row_map, void* part_ws, size_t part_ws_bytes,
                                       moe_stream_t stream) {
    MOE_REQUIRE(S_rows >= 0 && K > 0 && N > 0 && E_l > 0 && E_l <= GG_MAXG, MOE_ERR_INVALID, "grouped_gemm_mapped: bad shape");
    MOE_REQUIRE(act >= EPI_NONE && act <= EPI_SWIGLU, MOE_ERR_INVALID, "grouped_gemm_mapped: activation %d", act);
    MOE_REQUIRE(K % 64 == 0 && N % 8 == 0, MOE_ERR_UNSUPPORTED, "grouped_gemm_mapped: needs K %% 64 == 0 and N %% 8 == 0 (K=%d N=%d)", K, N);
    MOE_REQUIRE(a_rows >= 0 && out_rows >= 0, MOE_ERR_INVALID, "grouped_gemm_mapped: negative buffer rows");
    // gathered rows are addressed with 32-bit byte offsets from a_base
    MOE_REQUIRE(!a_row_map || (unsigned long long)a_rows * (unsigned long long)K * 2ull < (1ull << 32), MOE_ERR_UNSUPPORTED,
                "grouped_gemm_mapped: the gathered buffer must be smaller than 4 GiB (%d rows of %d)", a_rows, K);
    if (S_rows == 0) return MOE_OK;
    MOE_REQUIRE(a_base && packed && expert_cnt && out, MOE_ERR_INVALID, "grouped_gemm_mapped: null pointer");
    GemmParams p{};
    p.A = (const uint8_t*)a_base; p.B = (const uint8_t*)packed; p.C = out; p.cnt = expert_cnt;
    p.a_map = a_row_map; p.c_map = c_row_map;
    p.E_l = E_l; p.K = K; p.N = N; p.ldc = N; p.S_rows = S_rows;
    p.Npad = round_up(act == EPI_SWIGLU ? 2 * N : N, GG_BN);
    return launch_gemm<false>(p, act, (hipStream_t)stream, part_ws, part_ws_bytes);
}

extern "C" int moe_grouped_gemm_mapped_gated(const void* a_base, int a_rows, const int32_t* a_row_map, const void* packed,
                                             const int32_t* expert_cnt, int S_rows, int K, int N, int E_l, const float* row_gate,
                                             void* out, int out_rows, const int32_t* c_row_map, void* part_ws, size_t part_ws_bytes,
                                             moe_stream_t stream) {
    MOE_REQUIRE(S_rows >= 0 && K > 0 && N > 0 && E_l > 0 && E_l <= GG_MAXG, MOE_ERR_INVALID, "grouped_gemm_mapped_gated: bad shape");
    MOE_REQUIRE(K % 64 == 0 && N % 8 == 0, MOE_ERR_UNSUPPORTED, "grouped_gemm_mapped_gated: needs K %% 64 == 0 and N %% 8 == 0 (K=%d N=%d)", K, N);
    MOE_REQUIRE(a_rows >= 0 && out_rows >= 0, MOE_ERR_INVALID, "grouped_gemm_mapped_gated: negative buffer rows");
    MOE_REQUIRE(!a_row_map || (unsigned long long)a_rows * (unsigned long long)K * 2ull < (1ull << 32), MOE_ERR_UNSUPPORTED,
                "grouped_gemm_mapped_gated: the gathered buffer must be smaller than 4 GiB (%d rows of %d)", a_rows, K);
    if (S_rows == 0) return MOE_OK;
    MOE_REQUIRE(a_base && packed && expert_cnt && out && row_gate, MOE_ERR_INVALID, "grouped_gemm_mapped_gated: null pointer");
    GemmParams p{};
    p.A = (const uint8_t*)a_base; p.B = (const uint8_t*)packed; p.C = out; p.cnt = expert_cnt;
    p.a_map = a_row_map; p.c_map = c_row_map; p.row_scale = row_gate;
    p.E_l = E_l; p.K = K; p.N = N; p.ldc = N; p.S_rows = S_rows;
    p.Npad = round_up(N, GG_BN);
    return launch_gemm<false>(p, EPI_GATE, (hipStream_t)stream, part_ws, part_ws_bytes);
}

extern "C" int moe_grouped_gemm_act_keep(const void* a_base, int a_rows, const int32_t* a_row_map, const void* packed,
                                         const int32_t* expert_cnt, int S_rows, int K, int N, int E_l, int act, void* out,
                                         void* pre_act, void* part_ws, size_t part_ws_bytes, moe_stream_t stream) {
    MOE_REQUIRE(S_rows >= 0 && K > 0 && N > 0 && E_l > 0 && E_l <= GG_MAXG, MOE_ERR_INVALID, "grouped_gemm_act_keep: bad shape");
    MOE_REQUIRE(act > EPI_NONE && act <= EPI_SWIGLU, MOE_ERR_INVALID, "grouped_gemm_act_keep: activation %d", act);
    MOE_REQUIRE(K % 64 == 0 && N % 8 == 0, MOE_ERR_UNSUPPORTED, "grouped_gemm_act_keep: needs K %% 64 == 0 and N %% 8 == 0 (K=%d N=%d)", K, N);
    MOE_REQUIRE(a_rows >= 0, MOE_ERR_INVALID, "grouped_gemm_act_keep: negative buffer rows");
    MOE_REQUIRE(!a_row_map || (unsigned long long)a_rows * (unsigned long long)K * 2ull < (1ull << 32), MOE_ERR_UNSUPPORTED,
                "grouped_gemm_act_keep: the gathered buffer must be smaller than 4 GiB (%d rows of %d)", a_rows, K);
    if (S_rows == 0) return MOE_OK;
    MOE_REQUIRE(a_base && packed && expert_cnt && out && pre_act, MOE_ERR_INVALID, "grouped_gemm_act_keep: null pointer");
    GemmParams p{};
    p.A = (const uint8_t*)a_base; p.B = (const uint8_t*)packed; p.C = out; p.C2 = pre_act; p.cnt = expert_cnt;
    p.a_map = a_row_map;
    p.E_l = E_l; p.K = K; p.N = N; p.ldc = N; p.S_rows = S_rows;
    p.Npad = round_up(act == EPI_SWIGLU ? 2 * N : N, GG_BN);
    return launch_gemm<false>(p, act, (hipStream_t)stream, part_ws, part_ws_bytes);
}

extern "C" int moe_grouped_mlp(const void* tokens, const int32_t* expert_cnt, int dtype, int S_rows, int H, int F, int E_l,
                               int act, const void* w1, const void* w_up, const void* w2, void* hidden_ws, void* out,
                               moe_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    MOE_REQUIRE(S_rows >= 0 && H > 0 && F > 0 && E_l > 0 && E_l <= GG_MAXG, MOE_ERR_INVALID, "grouped_mlp: bad shape");
    MOE_REQUIRE(act == EPI_GELU || act == EPI_SILU || act == EPI_SWIGLU || act == EPI_NONE, MOE_ERR_INVALID,
                "grouped_mlp: activation %d", act);
    if (S_rows == 0) return MOE_OK;
    MOE_REQUIRE(tokens && expert_cnt && w1 && w2 && hidden_ws && out, MOE_ERR_INVALID, "grouped_mlp: null pointer");
    if (dtype == MOE_F32) {
        MOE_REQUIRE(act != EPI_SWIGLU || w_up, MOE_ERR_INVALID, "grouped_mlp: swiglu needs w_up");
        int rc = launch_f32((const float*)tokens, (const float*)w1, (const float*)w_up, (float*)hidden_ws, expert_cnt, E_l, H,
                            F, S_rows, act, s);
        if (rc) return rc;
        return launch_f32((const float*)hidden_ws, (const float*)w2, nullptr, (float*)out, expert_cnt, E_l, F, H, S_rows,
                          EPI_NONE, s);
    }
    MOE_REQUIRE(dtype == MOE_BF16, MOE_ERR_INVALID, "grouped_mlp: dtype %d", dtype);
    MOE_REQUIRE(w_up == nullptr, MOE_ERR_INVALID, "grouped_mlp: bf16 takes gate/up interleaved in w1 (w_up must be NULL)");
    MOE_REQUIRE(H % 64 == 0 && F % 64 == 0, MOE_ERR_UNSUPPORTED, "grouped_mlp: bf16 needs H, F multiples of 64 (H=%d F=%d)", H, F);
    GemmParams p{};
    p.A = (const uint8_t*)tokens; p.B = (const uint8_t*)w1; p.C = hidden_ws; p.cnt = expert_cnt;
    p.E_l = E_l; p.K = H; p.N = F; p.ldc = F; p.S_rows = S_rows;
    p.Npad = round_up(act == EPI_SWIGLU ? 2 * F : F, GG_BN);
    int rc = launch_gemm<false>(p, act, s);
    if (rc) return rc;
    GemmParams q{};
    q.A = (const uint8_t*)hidden_ws; q.B = (const uint8_t*)w2; q.C = out; q.cnt = expert_cnt;
    q.E_l = E_l; q.K = F; q.N = H; q.Npad = round_up(H, GG_BN); q.ldc = H; q.S_rows = S_rows;
    return launch_gemm<false>(q, EPI_NONE, s);
}

static int launch_quantize(const void* x_bf16, const int32_t* src_map, int rows, int cols, uint8_t* q, float* scale,
                           const int32_t* n_rows_dev, hipStream_t s) {
    const int blocks = min(ceil_div(rows, 4), 65535 * 8);
    const int nv = ceil_div(cols / 8, WAVE);  // 16-byte vectors per lane
#define GG_Q(NVv) quantize_rows_fp8_kernel<NVv><<<blocks, 256, 0, s>>>((const bf16_t*)x_bf16, rows, cols, q, scale, n_rows_dev, src_map)
    if (nv <= 2) GG_Q(2);
    else if (nv <= 4) GG_Q(4);
    else if (nv <= 8) GG_Q(8);
    else if (nv <= 16) GG_Q(16);
    else GG_Q(0);
#undef GG_Q
    return moe_check_launch("quantize_rows_fp8");
}

extern "C" int moe_quantize_rows_fp8(const void* x_bf16, int rows, int cols, uint8_t* q, float* scale,
                                     const int32_t* n_rows_dev, moe_stream_t stream) {
    MOE_REQUIRE(rows >= 0 && cols > 0 && cols % 8 == 0, MOE_ERR_INVALID, "quantize_rows_fp8: cols must be a multiple of 8");
    if (rows == 0) return MOE_OK;
    MOE_REQUIRE(x_bf16 && q && scale, MOE_ERR_INVALID, "quantize_rows_fp8: null pointer");
    return launch_quantize(x_bf16, nullptr, rows, cols, q, scale, n_rows_dev, (hipStream_t)stream);
}

// The two GEMMs of the fp8 SwiGLU expert on quantised rows (xq codes gathered through a_map, xs their scales in GEMM row
// order): gate/up + SwiGLU with the hidden activation quantised in the epilogue (codes hq, one E8M0 scale byte per row and
// 32 columns in hscale), then the down projection, which takes those bytes as the scale operand of its MFMAs; row_gate
// (nullable) multiplies the result rows.
static int fp8_mlp_gemms(const uint8_t* xq, const int32_t* a_map, const float* xs, const int32_t* expert_cnt, int S_rows, int H, int F,
                         int E_l, const uint8_t* wgu_packed, const float* sg, const float* su, const uint8_t* wd_packed,
                         const float* sd, uint8_t* hq_ws, uint8_t* hscale_ws, const float* row_gate, void* out,
                         const int32_t* c_row_map, void* part_ws, size_t part_ws_bytes, hipStream_t s) {
    GemmParams p{};
    p.A = xq; p.B = wgu_packed; p.C = hq_ws; p.cnt = expert_cnt; p.row_scale = xs; p.col_scale = sg; p.col_scale2 = su;
    p.a_map = a_map; p.c_bscale = hscale_ws; p.bs_pitch = F / 32;
    p.E_l = E_l; p.K = H; p.N = F; p.Npad = round_up(2 * F, GG_BN); p.ldc = F; p.S_rows = S_rows; p.ncs = F;
    int rc = launch_gemm<true>(p, EPI_SWIGLU, s, part_ws, part_ws_bytes);
    if (rc) return rc;
    GemmParams q{};
    q.A = hq_ws; q.B = wd_packed; q.C = out; q.cnt = expert_cnt; q.row_scale = row_gate; q.col_scale = sd;
    q.c_map = c_row_map; q.a_bscale = hscale_ws; q.bs_pitch = F / 32;
    q.E_l = E_l; q.K = F; q.N = H; q.Npad = round_up(H, GG_BN); q.ldc = H; q.S_rows = S_rows; q.ncs = H;
    return launch_gemm<true>(q, EPI_NONE, s, part_ws, part_ws_bytes);
}

extern "C" int moe_grouped_mlp_fp8_mapped(const void* a_base_bf16, int a_rows, const int32_t* a_row_map,
                                          const int32_t* expert_cnt, int S_rows, int H, int F, int E_l,
                                          const uint8_t* wgu_packed, const float* sg, const float* su,
                                          const uint8_t* wd_packed, const float* sd, uint8_t* xq_ws, float* xs_ws,
                                          uint8_t* hq_ws, uint8_t* hscale_ws, const float* row_gate, void* out, int out_rows,
                                          const int32_t* c_row_map, void* part_ws, size_t part_ws_bytes, moe_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    MOE_REQUIRE(S_rows >= 0 && H > 0 && F > 0 && E_l > 0 && E_l <= GG_MAXG, MOE_ERR_INVALID, "grouped_mlp_fp8: bad shape");
    MOE_REQUIRE(H % 128 == 0 && F % 128 == 0, MOE_ERR_UNSUPPORTED, "grouped_mlp_fp8: needs H, F multiples of 128 (H=%d F=%d)", H, F);
    MOE_REQUIRE(a_rows >= 0 && out_rows >= 0, MOE_ERR_INVALID, "grouped_mlp_fp8: negative buffer rows");
    MOE_REQUIRE((unsigned long long)S_rows * (unsigned long long)(F / 32) < (1ull << 32), MOE_ERR_UNSUPPORTED,
                "grouped_mlp_fp8: the block scales must stay under 4 GiB");
    if (S_rows == 0) return MOE_OK;
    MOE_REQUIRE(a_base_bf16 && expert_cnt && wgu_packed && sg && su && wd_packed && sd && xq_ws && xs_ws && hq_ws && hscale_ws && out,
                MOE_ERR_INVALID, "grouped_mlp_fp8: null pointer");
    // the row quantisation reads every input row once anyway: with a map it reads it where the transfer left it
    int rc = launch_quantize(a_base_bf16, a_row_map, S_rows, H, xq_ws, xs_ws, nullptr, s);
    if (rc) return rc;
    return fp8_mlp_gemms(xq_ws, nullptr, xs_ws, expert_cnt, S_rows, H, F, E_l, wgu_packed, sg, su, wd_packed, sd, hq_ws, hscale_ws,
                         row_gate, out, c_row_map, part_ws, part_ws_bytes, s);
}

extern "C" int moe_grouped_mlp_fp8(const void* tokens_bf16, const int32_t* expert_cnt, int S_rows, int H, int F, int E_l,
                                   const uint8_t* wgu_packed, const float* sg, const float* su, const uint8_t* wd_packed,
                                   const float* sd, uint8_t* xq_ws, float* xs_ws, uint8_t* hq_ws, uint8_t* hscale_ws, void* out,
                                   moe_stream_t stream) {
    return moe_grouped_mlp_fp8_mapped(tokens_bf16, S_rows, nullptr, expert_cnt, S_rows, H, F, E_l, wgu_packed, sg, su, wd_packed,
                                      sd, xq_ws, xs_ws, hq_ws, hscale_ws, nullptr, out, S_rows, nullptr, nullptr, 0, stream);
}

extern "C" int moe_pack_tokens_fp8(const void* x_bf16, int T, int H, const int32_t* topk_idx, const int32_t* pos, int k, int E_l,
                                   const int32_t* dst_sizes, const int32_t* dst_offsets, int W, int M, uint8_t* send_q,
                                   float* send_scale, int32_t* status, moe_stream_t stream) {
    return moe_pack_tokens_fp8_gated(x_bf16, T, H, topk_idx, pos, nullptr, k, E_l, dst_sizes, dst_offsets, W, M, send_q, send_scale,
                                     nullptr, status, stream);
}

extern "C" int moe_pack_tokens_fp8_gated(const void* x_bf16, int T, int H, const int32_t* topk_idx, const int32_t* pos,
                                         const float* gate, int k, int E_l, const int32_t* dst_sizes, const int32_t* dst_offsets,
                                         int W, int M, uint8_t* send_q, float* send_scale, float* send_gate, int32_t* status,
                                         moe_stream_t stream) {
    MOE_REQUIRE((gate == nullptr) == (send_gate == nullptr), MOE_ERR_INVALID, "pack_tokens_fp8: gate and send_gate go together");
    MOE_REQUIRE(T >= 0 && H > 0 && H % 8 == 0 && W > 0 && M >= 1 && E_l > 0, MOE_ERR_INVALID, "pack_tokens_fp8: bad shape");
    MOE_REQUIRE(k >= 1 && k <= MOE_MAX_TOPK, MOE_ERR_UNSUPPORTED, "pack_tokens_fp8: topk=%d outside [1,%d]", k, MOE_MAX_TOPK);
    MOE_REQUIRE((long long)W * M + T < (1ll << 31), MOE_ERR_UNSUPPORTED, "pack_tokens_fp8: W*M + T too large");
    MOE_REQUIRE(send_q && send_scale && dst_sizes && dst_offsets, MOE_ERR_INVALID, "pack_tokens_fp8: null pointer");
    MOE_REQUIRE(T == 0 || (x_bf16 && topk_idx && pos), MOE_ERR_INVALID, "pack_tokens_fp8: null pointer");
    const int n_units = T + ceil_div(W * M, PACKQ_ZR);
    const int blocks = min(ceil_div(n_units, 4), 65535 * 8);
    const int nv = ceil_div(H / 8, WAVE);
    hipStream_t s = (hipStream_t)stream;
#define GG_PQ(NVv) pack_tokens_fp8_kernel<NVv><<<blocks, 256, 0, s>>>((const bf16_t*)x_bf16, T, H, topk_idx, pos, dst_sizes, dst_offsets, k, E_l, W, M, send_q, send_scale, status, gate, send_gate)
    if (nv <= 2) GG_PQ(2);
    else if (nv <= 4) GG_PQ(4);
    else if (nv <= 8) GG_PQ(8);
    else if (nv <= 16) GG_PQ(16);
    else GG_PQ(0);
#undef GG_PQ
    return moe_check_launch("pack_tokens_fp8");
}

extern "C" int moe_grouped_mlp_fp8_q_mapped(const uint8_t* a_q, const float* a_scale, int a_rows, const int32_t* a_row_map,
                                            const int32_t* expert_cnt, int S_rows, int H, int F, int E_l,
                                            const uint8_t* wgu_packed, const float* sg, const float* su,
                                            const uint8_t* wd_packed, const float* sd, float* xs_ws, uint8_t* hq_ws,
                                            uint8_t* hscale_ws, const float* row_gate, void* out, int out_rows,
                                            const int32_t* c_row_map, void* part_ws, size_t part_ws_bytes, moe_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    MOE_REQUIRE(S_rows >= 0 && H > 0 && F > 0 && E_l > 0 && E_l <= GG_MAXG, MOE_ERR_INVALID, "grouped_mlp_fp8_q: bad shape");
    MOE_REQUIRE(H % 128 == 0 && F % 128 == 0, MOE_ERR_UNSUPPORTED, "grouped_mlp_fp8_q: needs H, F multiples of 128 (H=%d F=%d)", H, F);
    MOE_REQUIRE(a_rows >= 0 && out_rows >= 0, MOE_ERR_INVALID, "grouped_mlp_fp8_q: negative buffer rows");
    MOE_REQUIRE(!a_row_map || (unsigned long long)a_rows * (unsigned long long)H < (1ull << 32), MOE_ERR_UNSUPPORTED,
                "grouped_mlp_fp8_q: the gathered buffer must be smaller than 4 GiB (%d rows of %d)", a_rows, H);
    MOE_REQUIRE((unsigned long long)S_rows * (unsigned long long)(F / 32) < (1ull << 32), MOE_ERR_UNSUPPORTED,
                "grouped_mlp_fp8_q: the block scales must stay under 4 GiB");
    if (S_rows == 0) return MOE_OK;
    MOE_REQUIRE(a_q && a_scale && expert_cnt && wgu_packed && sg && su && wd_packed && sd && xs_ws && hq_ws && hscale_ws && out,
                MOE_ERR_INVALID, "grouped_mlp_fp8_q: null pointer");
    // the row scales in the order of the GEMM's rows (the codes themselves are gathered by the GEMM as it loads them)
    gather_scale_kernel<<<ceil_div(S_rows, 256), 256, 0, s>>>(a_scale, a_row_map, S_rows, xs_ws);
    return fp8_mlp_gemms(a_q, a_row_map, xs_ws, expert_cnt, S_rows, H, F, E_l, wgu_packed, sg, su, wd_packed, sd, hq_ws, hscale_ws,
                         row_gate, out, c_row_map, part_ws, part_ws_bytes, s);
}

// ---- backward pass entry points --------------------------------------------------------------------------------------
extern "C" int moe_prepack_weights_transposed(const void* w, const void* w_up, int dtype, int E_l, int K, int N, void* packed,
                                              moe_stream_t stream) {
    MOE_REQUIRE(dtype == MOE_BF16, MOE_ERR_INVALID, "prepack_weights_transposed: bf16 only (dtype %d)", dtype);
    MOE_REQUIRE(E_l > 0 && K > 0 && N > 0 && w && packed, MOE_ERR_INVALID, "prepack_weights_transposed: bad arguments");
    MOE_REQUIRE(N % 64 == 0 && K % 8 == 0, MOE_ERR_UNSUPPORTED,
                "prepack_weights_transposed: needs N %% 64 == 0 and K %% 8 == 0 (K=%d N=%d)", K, N);
    const int Kpad = round_up(K, GG_BN);
    prepack_t_kernel<uint16_t><<<dim3(1024, E_l), 256, 0, (hipStream_t)stream>>>((const uint16_t*)w, (const uint16_t*)w_up,
                                                                               (uint16_t*)packed, K, N, Kpad);
    return moe_check_launch("prepack_weights_transposed");
}

extern "C" size_t moe_dw_workspace_bytes(int S_rows, int E_l, int K, int N) {
    if (S_rows < 0 || E_l <= 0 || K <= 0 || N <= 0) return 0;
    const size_t spad = (size_t)round_up(S_rows, 64) + (size_t)64 * E_l;
    return spad * ((size_t)K + (size_t)round_up(N, GG_BN)) * 2;
}

extern "C" int moe_grouped_gemm_dw(const void* x, const void* dy, const int32_t* expert_cnt, int dtype, int S_rows, int K, int N,
                                   int E_l, int split_F, void* dw, void* ws, size_t ws_bytes, moe_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
    MOE_REQUIRE(S_rows >= 0 && K > 0 && N > 0 && E_l > 0 && E_l <= GG_MAXG, MOE_ERR_INVALID, "grouped_gemm_dw: bad shape");
    MOE_REQUIRE(expert_cnt && dw && (S_rows == 0 || (x && dy)), MOE_ERR_INVALID, "grouped_gemm_dw: null pointer");
    MOE_REQUIRE(split_F == 0 || (dtype == MOE_BF16 && split_F % 32 == 0 && N == 2 * split_F), MOE_ERR_INVALID,
                "grouped_gemm_dw: split_F=%d needs bf16, split_F %% 32 == 0 and N == 2 split_F", split_F);
    if (dtype == MOE_F32) {
        grouped_dw_f32_kernel<<<dim3(ceil_div(N, 64), ceil_div(K, 64), E_l), 256, 0, s>>>((const float*)x, (const float*)dy, expert_cnt,
                                                                                       E_l, K, N, S_rows, (float*)dw);
        return moe_check_launch("grouped_gemm_dw_f32");
    }
    MOE_REQUIRE(dtype == MOE_BF16, MOE_ERR_INVALID, "grouped_gemm_dw: dtype %d", dtype);
    MOE_REQUIRE(N % 8 == 0 && K % 8 == 0, MOE_ERR_UNSUPPORTED, "grouped_gemm_dw: bf16 needs K, N multiples of 8 (K=%d N=%d)", K, N);
    MOE_REQUIRE(ws && ws_bytes >= moe_dw_workspace_bytes(S_rows, E_l, K, N), MOE_ERR_WORKSPACE, "grouped_gemm_dw: workspace %zu < %zu",
                ws_bytes, moe_dw_workspace_bytes(S_rows, E_l, K, N));
    const int spad = round_up(S_rows, 64) + 64 * E_l;  // upper bound of the padded row total, and the operands' pitch
    MOE_REQUIRE((unsigned long long)K * (unsigned long long)spad * 2ull < (1ull << 32), MOE_ERR_UNSUPPORTED,
                "grouped_gemm_dw: the transposed activations must stay under 4 GiB (%d x %d)", K, spad);
    const int Npad = round_up(N, GG_BN);
    uint16_t* xT = (uint16_t*)ws;                       // [K, spad]
    uint16_t* dyP = xT + (size_t)K * spad;              // [spad / 32][Npad][32]
    const int pblocks = spad / 64;
    dw_zero_empty_kernel<<<dim3(256, E_l), 256, 0, s>>>((uint4*)dw, expert_cnt, (size_t)K * N * 2 / 16, S_rows);
    if (S_rows > 0) {
        dw_operand_kernel<false><<<dim3(ceil_div(K, 64), pblocks), 256, 0, s>>>((const uint16_t*)x, expert_cnt, E_l, S_rows, K, xT, spad, 0, 0);
        dw_operand_kernel<true><<<dim3(Npad / 64, pblocks), 256, 0, s>>>((const uint16_t*)dy, expert_cnt, E_l, S_rows, N, dyP, spad, Npad, split_F);
        GemmParams p{};
        p.A = (const uint8_t*)xT; p.B = (const uint8_t*)dyP; p.C = dw; p.cnt = expert_cnt;
        p.E_l = E_l; p.K = spad; p.N = N; p.Npad = Npad; p.ldc = N; p.S_rows = K;
        p.dw_rows = K; p.dw_src_rows = S_rows; p.c_group_stride = (size_t)K * N;
        grouped_gemm_kernel<256, GG_BIG_NWM, EPI_NONE, false, false, true><<<num_cus(), GG_BIG_NWM * 2 * WAVE, 0, s>>>(p);
    }
    return moe_check_launch("grouped_gemm_dw");
}

extern "C" int moe_transpose_weights_f32(const float* w, int E_l, int K, int N, float* out, moe_stream_t stream) {
    MOE_REQUIRE(E_l > 0 && K > 0 && N > 0 && w && out, MOE_ERR_INVALID, "transpose_weights_f32: bad arguments");
    transpose_f32_kernel<<<dim3(ceil_div(N, 32), ceil_div(K, 32), E_l), 256, 0, (hipStream_t)stream>>>(w, out, K, N);
    return moe_check_launch("transpose_weights_f32");
}

extern "C" int moe_mlp_act_backward(const void* a1, const void* dh, int dtype, int rows, int F, int act, void* d_a1,
                                    moe_stream_t stream) {
    MOE_REQUIRE(rows >= 0 && F > 0, MOE_ERR_INVALID, "mlp_act_backward: bad shape");
    MOE_REQUIRE(dtype == MOE_BF16 || (dtype == MOE_F32 && act != EPI_SWIGLU), MOE_ERR_UNSUPPORTED,
                "mlp_act_backward: dtype %d with activation %d", dtype, act);
    MOE_REQUIRE(act == EPI_GELU || act == EPI_SILU || act == EPI_SWIGLU, MOE_ERR_INVALID, "mlp_act_backward: activation %d", act);
    MOE_REQUIRE(act != EPI_SWIGLU || F % 32 == 0, MOE_ERR_UNSUPPORTED, "mlp_act_backward: swiglu needs F %% 32 == 0");
    if (rows == 0) return MOE_OK;
    MOE_REQUIRE(a1 && dh && d_a1, MOE_ERR_INVALID, "mlp_act_backward: null pointer");
    const int blocks = (int)std::min<size_t>(((size_t)rows * F + 255) / 256, (size_t)num_cus() * 32);
    hipStream_t s = (hipStream_t)stream;
#define GG_ACTB(EPIv, Tv) act_backward_kernel<EPIv, Tv><<<blocks, 256, 0, s>>>((const Tv*)a1, (const Tv*)dh, (Tv*)d_a1, (size_t)rows, F)
    if (dtype == MOE_F32) {
        if (act == EPI_GELU) GG_ACTB(EPI_GELU, float);
        else GG_ACTB(EPI_SILU, float);
    } else if (act == EPI_GELU) GG_ACTB(EPI_GELU, bf16_t);
    else if (act == EPI_SILU) GG_ACTB(EPI_SILU, bf16_t);
    else GG_ACTB(EPI_SWIGLU, bf16_t);
#undef GG_ACTB
    return moe_check_launch("mlp_act_backward");
}
