// Ring / block attention for MI355X (gfx950, CDNA4): forward with online softmax across
// KV chunks resident in HBM, recompute backward, behind the C ABI of include/ltr_attn.h.
//
// Kernel map
//   fwd_bf16_kernel<D, RB>   S^T = K Q^T and O^T = V^T P^T on v_mfma_f32_32x32x16_bf16; a block of
//                        8 waves owns 256 * RB query rows, a wave 32 * RB of them, so a lane owns ONE query per row block:
//                        the row sums are in-lane reductions (no running max: the reference of the
//                        exponent moves only when a row sum leaves its safe range), and P^T leaves the
//                        first GEMM already in the B-operand layout of the second.  64-key K
//                        and V tiles go global -> LDS directly (no staging registers) into
//                        unpadded, XOR-swizzled, double-buffered tiles, one barrier per tile;
//                        the V^T operand is read with ds_read_b64_tr_b16.  The (O, LSE) merge
//                        with an earlier partial result is part of the epilogue.
//                        fwd_bf16_kernel<64, 2>: two 32-row blocks per wave (512 rows per block, 64-key tiles): every K / V
//                        operand read from LDS feeds two MFMAs (chosen by the host, or forced with LTR_FWD_ROWS_512).
//   fwd_f32_mfma_kernel<D, KS>  fp32 I/O and arithmetic on v_mfma_f32_32x32x2_f32: the forward of the 1e-4 cases (the reference's
//                        acceptance dtype) on the matrix pipe; KS key shares per 32-row group for launches with few rows.
//   fwd_f32_kernel<D>    the same in scalar fp32 (no MFMA): kept as the fallback, reached with LTR_FWD_F32_SCALAR.
//   delta_kernel         DELTA = rowsum(dO * O).
//   bwd_dkdv_kernel<D, KW>  a block of 8 waves owns 128 * KW keys of one kv head and loops over the
//                        query heads of the GQA group and over 64-row query tiles taken from
//                        lists (fully visible / partly masked) built once in LDS.  Two waves
//                        share each 32-key slice: one computes S, P and dV^T, the other dP,
//                        dS and dK^T one tile behind, P handed over through LDS.  Q / dO tiles
//                        go global -> LDS directly into three swizzled buffers, one barrier
//                        per tile; K, V operands and the dK^T / dV^T accumulators stay in
//                        registers for the whole block.
//                        bwd_dkdv_kernel<64, 2>: two 32-key halves per wave (256 keys per block): every Q / dO operand
//                        read from LDS feeds two MFMAs, and a block's transfers and per-step costs are spread over
//                        twice the matrix work.  The registers allow it at head dim 64 only; chosen by the host
//                        when the blocks are long and still many (or forced with LTR_DKDV_KEYS_256).
//   bwd_dq_kernel<D, RB> forward-shaped: a block owns 256 * RB query rows, loops over K/V tiles
//                        (same direct-to-LDS tiles as the forward), recomputes S and dP and
//                        accumulates dQ^T in registers.  No atomics anywhere: results are
//                        bitwise reproducible.  bwd_dq_kernel<64, 2>: two 32-row blocks per wave (a lane owns two
//                        query rows): every K / V operand read from LDS feeds two MFMAs; head dim 64 only, chosen by the
//                        host when the wider blocks still fill the device (or forced with LTR_DQ_ROWS_512).
//   bwd_dq_f32_mfma_kernel<D, KS>, bwd_dkdv_f32_mfma_kernel<D>
//                        the fp32 backward on v_mfma_f32_32x32x2_f32 (see there).
//   bwd_dq_f32_kernel<D>, bwd_dkdv_f32_kernel<D, DV>
//                        the same backward in scalar fp32 (no MFMA): the fallback, reached with LTR_BWD_F32_SCALAR.
//   The tile loops of the bf16 kernels are unrolled over their LDS buffers (or, where registers are short,
//   keep per-lane LDS addresses in registers): no address arithmetic is left between the MFMAs.
//   RoPE: with LTR_ROPE_Q the forward rotates each q row in its operand registers (rope_rotate8) and can store the
//   rotated row; with LTR_ROPE_DQ the dQ kernel's epilogue rotates dQ by the conjugate angles (rope_conj4).
//   Block scheduling under a causal mask: a forward / dQ block takes a late q tile and its early counterpart when the
//   host says so (q_tile_slots; every other block in the opposite order, so that equal blocks do not all change tiles
//   at once), and the dK/dV kernel's chunk table is sorted by position (longest blocks first).
//   ltr_attn_bwd_noalloc keeps its DELTA workspace in the fixed __device__ array `scratch` (see there).
//
// MFMA 32x32x16 operand layout used throughout (lane l, i = l % 32, h = l / 32):
//   A[i][8h .. 8h+7], B[8h .. 8h+7][i], C[8*(r/4) + 4h + r%4][i] for accumulator register r.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <math.h>
#include <stdio.h>
#include <type_traits>
#include <atomic>
#include <algorithm>
#include "ltr_attn.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

#define LTR_LOG2E 1.4426950408889634f
#define LTR_LN2 0.6931471805599453f

struct ChunkDev {
    const void *k;
    const void *v;
    float *dk;
    float *dv;
    int sk;
    int pos0;
};

struct FwdParams {
    const void *q;
    void *o;
    float *lse;
    int B, Hq, Hkv, n_rep;
    int Sq, n_qtiles;
    int n_slots;           // q tiles are handed out in slots: n_qtiles of one tile, or (n_qtiles + 1) / 2 of two (see q_tile_slots)
    long long qs[3], os[3], ks[3], vs[3];
    int q_pos0[2];
    int q_split;
    float scale;
    unsigned flags;
    int o_f32;
    int n_chunks;
    const float *rope;     // LTR_ROPE_Q: (cos, sin) rows, D floats per position, row 0 = position rope_pos0
    int rope_pos0;
    void *q_rot;           // optional bf16 output: the rotated q
    long long qrs[3];
    ChunkDev chunk[LTR_MAX_CHUNKS];
};

struct BwdParams {
    const void *q;
    const void *d_o;
    const float *lse;
    float *delta;      // read; written by the dQ kernel with LTR_DELTA_FROM_O
    const void *o;     // bf16 forward output, read with LTR_DELTA_FROM_O only
    long long os_[3];
    void *dq;          // fp32 accumulator, or bf16 result with LTR_DQ_BF16
    int B, Hq, Hkv, n_rep;
    int Sq, n_qtiles;
    long long qs[3], dos[3], dqs[3], ks[3], vs[3], dks[3], dvs[3];
    int q_pos0[2];
    int q_split;
    float scale;
    unsigned flags;
    int n_chunks;
    int tiles_total;  // key tiles over all chunks
    int n_slots;      // slots of 256-row q tiles of the dQ kernel (see q_tile_slots)
    const float *rope;     // LTR_ROPE_DQ: (cos, sin) rows, D floats per position, row 0 = position rope_pos0
    int rope_pos0;
    ChunkDev chunk[LTR_MAX_CHUNKS];
};

struct DeltaParams {
    const void *o;
    const void *d_o;
    float *delta;
    int B, Hq, D, Sq;
    long long os[3], dos[3];
    int o_f32, do_f32;
};

__device__ __forceinline__ int q_position(int row, int split, int p0, int p1) {
    return row < split ? p0 + row : p1 + (row - split);
}

// min and max global position over local rows [r0, r1] (inclusive, r0 <= r1)
__device__ __forceinline__ void q_pos_range(int r0, int r1, int split, int p0, int p1, int &lo, int &hi) {
    int a = q_position(r0, split, p0, p1), b = q_position(r1, split, p0, p1);
    lo = min(a, b);
    hi = max(a, b);
    if (r0 < split && r1 >= split) {  // tile straddles the two segments
        int c = q_position(split - 1, split, p0, p1), d = q_position(split, split, p0, p1);
        lo = min(lo, min(c, d));
        hi = max(hi, max(c, d));
    }
}

// both halves of the wave end up with combine(x[l], x[l ^ 32])
__device__ __forceinline__ float xhalf_max(float x) {
    unsigned u = __float_as_uint(x);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xhalf_sum(float x) {
    unsigned u = __float_as_uint(x);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// ds_read_b64_tr_b16: within each group of 16 lanes, lane i receives as element e the
// 16-bit value that lane (4e + i/4) of the group addressed at position i % 4.  With lane s
// of a group pointing at M[k0 + s/4][n0 + 4*(s%4)] of a row-major tile, lane i receives
// M[k0 + 0..3][n0 + i]: four consecutive rows of one column, i.e. the MFMA K-dim packing.
__device__ __forceinline__ i16x4 lds_read_tr16(const __bf16 *p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((i16x4 __attribute__((address_space(3))) *)(p));
}

// Unpadded row-major LDS tile of D bf16 per row whose 16-byte chunks are XOR-swizzled: chunk c of row r
// lives at chunk position c ^ lds_swz<D>(r).  LDS has 64 banks of 4 bytes; a 128-bit read is served 16
// lanes at a time and a 64-bit (transpose) read 32 lanes at a time.  With this permutation both the MFMA
// operand read (16 consecutive rows, same logical chunk) and the transpose read (4 consecutive rows x 4
// consecutive chunks) touch every bank exactly once, and so does the staging store (one row per 16 lanes).
template <int D>
__device__ __forceinline__ int lds_swz(int row) {
    return D == 128 ? (((row & 3) << 2) | ((row >> 2) & 3)) : ((((row >> 1) & 1) << 2) | ((row >> 2) & 3));
}

template <int D>
__device__ __forceinline__ int lds_swz_off(int row, int chunk) {   // element offset of (row, 16-byte chunk)
    return row * D + ((chunk ^ lds_swz<D>(row)) << 3);
}

// 8 K-dim values for an MFMA operand whose K index runs over the ROWS of a row-major LDS
// tile: rows {k0 + 4h + 0..3} and {k0 + 8 + 4h + 0..3} at column n_base + (l % 32).
// This row set is the one the accumulator registers 8b..8b+7 of a 32x32 MFMA result
// hold (rows 16b + 4h + 0..3 and 16b + 8 + 4h + 0..3), so a result tile can feed the
// next GEMM as an operand without leaving registers.
// (tile = swizzled tile, see lds_swz)
template <int D>
__device__ __forceinline__ bf16x8 lds_operand_tr_swz(const __bf16 *tile, int k0, int n_base, int lane) {
    const int li = lane & 15, g = lane >> 4;
    const int hh = g >> 1;
    const int col = n_base + ((g & 1) << 4) + ((li & 3) << 2);
    const int row = k0 + 4 * hh + (li >> 2);
    i16x4 lo = lds_read_tr16(tile + lds_swz_off<D>(row, col >> 3) + (col & 7));
    i16x4 hi = lds_read_tr16(tile + lds_swz_off<D>(row + 8, col >> 3) + (col & 7));
    union {
        struct { i16x4 a, b; } s;
        bf16x8 v;
    } u;
    u.s.a = lo;
    u.s.b = hi;
    return u.v;
}

// 16 bytes per lane from global memory straight into LDS: lane l's data lands at LDS byte address lds_byte_addr + 16*l
// (wave-uniform; lds_address() of a __shared__ object plus an offset).  No staging registers, no LDS store pass.  Written as inline assembly so that the compiler
// does not track the transfer: with the builtin it makes the next LDS read of ANY address wait for vmcnt(0),
// which would expose the whole global-memory latency in the middle of a tile.  The transfer is only complete
// after tile_barrier() (the only place that waits for it); nothing may read the destination before that.
__device__ __forceinline__ unsigned lds_address(const void *shared_object) {
    return (unsigned)(uintptr_t)(__attribute__((address_space(3))) const void *)shared_object;
}

__device__ __forceinline__ void global_to_lds_b128(const void *gptr, unsigned lds_byte_addr_uniform) {
    const unsigned lds_addr = __builtin_amdgcn_readfirstlane(lds_byte_addr_uniform);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(lds_addr) : "memory", "m0");
}

// End of a tile: wait for every outstanding tile transfer and LDS access of this wave, then the block
// barrier.  The wait is the s_waitcnt builtin (vmcnt(0) lgkmcnt(0), expcnt left alone) so that the compiler's
// own counter bookkeeping knows that nothing is pending afterwards.
__device__ __forceinline__ void tile_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0070);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

__device__ __forceinline__ bf16x8 as_bf16x8(uint4 x) {
    union { uint4 u; bf16x8 v; } c;
    c.u = x;
    return c.v;
}

// Rotary position embedding of 8 consecutive elements (4 adjacent (re, im) pairs) of one row: f0, f1 hold the pairs'
// (cos, sin).  The arithmetic of apply_rotary_emb (layers/layers.py:44-70) as the streaming kernel of ltr_rope_apply does
// it: fp32 complex multiply with the four products rounded separately, result rounded to bf16 - so a row rotated here has
// the bits that the separate pass would have written.
__device__ __forceinline__ bf16x8 rope_rotate8(bf16x8 x, f32x4 f0, f32x4 f1) {
#pragma clang fp contract(off)
    const float cs[4] = {f0[0], f0[2], f1[0], f1[2]}, sn[4] = {f0[1], f0[3], f1[1], f1[3]};
    bf16x8 out;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float re = (float)x[2 * i], im = (float)x[2 * i + 1];
        const float rr = re * cs[i], ii = im * sn[i];
        const float ri = re * sn[i], ir = im * cs[i];
        out[2 * i] = (__bf16)(rr - ii);
        out[2 * i + 1] = (__bf16)(ri + ir);
    }
    return out;
}

// Gradient of that rotation: 4 consecutive fp32 elements (2 pairs) times the CONJUGATE angles; f = (cos, sin, cos, sin).
__device__ __forceinline__ f32x4 rope_conj4(f32x4 v, f32x4 f) {
#pragma clang fp contract(off)
    f32x4 out;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const float re = v[2 * i], im = v[2 * i + 1], c = f[2 * i], sn = f[2 * i + 1];
        out[2 * i] = re * c + im * sn;
        out[2 * i + 1] = im * c - re * sn;
    }
    return out;
}

struct PackedTile {   // 16 bf16 values of one lane's 32x32 tile column, as the two B operands of K = 16
    unsigned u[8];
};

__device__ __forceinline__ unsigned pack2_bf16(float a, float b) {
    bf16x2 t;
    t[0] = (__bf16)a;
    t[1] = (__bf16)b;
    return __builtin_bit_cast(unsigned, t);
}

__device__ __forceinline__ bf16x8 operand_of(const PackedTile &t, int kb) {
    union { unsigned u[4]; bf16x8 v; } c;
    c.u[0] = t.u[4 * kb];
    c.u[1] = t.u[4 * kb + 1];
    c.u[2] = t.u[4 * kb + 2];
    c.u[3] = t.u[4 * kb + 3];
    return c.v;
}

// Two independent 32x32 accumulation chains over the head dimension (added to ra / rb as passed in), A operands from rows of swizzled LDS tiles
// (row pointers rowa / rowb, swizzle words swa / swb of those rows, already XOR-ed with the lane's half),
// B operands from registers.  The chains alternate so no MFMA waits for its predecessor, and the operand reads
// run PF steps ahead of the MFMAs that use them; sched_barrier pins that order (left alone, the scheduler sinks
// each read to just before its use and the full LDS latency is exposed at every step).
template <int D>
__device__ __forceinline__ void lds_gemm_pair(const __bf16 *rowa, int swa, const __bf16 *rowb, int swb,
                                              const bf16x8 (&ba)[D / 16], const bf16x8 (&bb)[D / 16],
                                              f32x16 &ra, f32x16 &rb) {
    constexpr int NK = D / 16, PF = 2;
    bf16x8 xa[PF + 1], xb[PF + 1];
#pragma unroll
    for (int i = 0; i < PF; i++) {
        xa[i] = *(const bf16x8 *)(rowa + (((2 * i) ^ swa) << 3));
        xb[i] = *(const bf16x8 *)(rowb + (((2 * i) ^ swb) << 3));
    }
#pragma unroll
    for (int kb = 0; kb < NK; kb++) {
        if (kb + PF < NK) {
            xa[(kb + PF) % (PF + 1)] = *(const bf16x8 *)(rowa + (((2 * (kb + PF)) ^ swa) << 3));
            xb[(kb + PF) % (PF + 1)] = *(const bf16x8 *)(rowb + (((2 * (kb + PF)) ^ swb) << 3));
        }
        __builtin_amdgcn_sched_barrier(0);
        ra = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[kb % (PF + 1)], ba[kb], ra, 0, 0, 0);
        rb = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xb[kb % (PF + 1)], bb[kb], rb, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
}

struct NoHook {
    __device__ __forceinline__ void operator()(int) const {}
};

// One 32x32 accumulation chain over the head dimension (added to r as passed in): A operands from row `row` of a
// swizzled LDS tile (sw = swizzle word of the row XOR the lane's half), B operands from registers.  hook(kb)
// is placed right after MFMA kb: independent arithmetic of the same wave written there issues while the matrix
// pipe works on that MFMA (a wave issues one instruction per ~5 clocks, an MFMA occupies the pipe for 32).
template <int D, class Hook = NoHook>
__device__ __forceinline__ void lds_gemm_chain(const __bf16 *row, int sw, const bf16x8 (&b)[D / 16], f32x16 &r,
                                               Hook hook = Hook()) {
    constexpr int NK = D / 16, PF = 2;
    bf16x8 x[PF + 1];
#pragma unroll
    for (int i = 0; i < PF; i++) x[i] = *(const bf16x8 *)(row + (((2 * i) ^ sw) << 3));
#pragma unroll
    for (int kb = 0; kb < NK; kb++) {
        if (kb + PF < NK) x[(kb + PF) % (PF + 1)] = *(const bf16x8 *)(row + (((2 * (kb + PF)) ^ sw) << 3));
        __builtin_amdgcn_sched_barrier(0);
        r = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x[kb % (PF + 1)], b[kb], r, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        hook(kb);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// acc[db] (32 x 32 tiles over the head dimension) += T^T-operand x B for NKB blocks of 16 tile rows starting at
// row0: the A operands are transpose reads of the swizzled LDS tile T (rows = contraction index), the B
// operands b[kb] come from registers.  Reads run PF MFMAs ahead, order pinned as in lds_gemm_pair; hook(step)
// is placed right after MFMA `step` (see lds_gemm_chain).
template <int D, int NKB, class Hook = NoHook>
__device__ __forceinline__ void lds_tr_gemm(const __bf16 *T, int row0, int lane, const bf16x8 (&b)[NKB],
                                            f32x16 (&acc)[D / 32], Hook hook = Hook()) {
    constexpr int ND = D / 32, N = NKB * ND, PF = 3;
    bf16x8 a[PF + 1];
#pragma unroll
    for (int i = 0; i < PF && i < N; i++) a[i] = lds_operand_tr_swz<D>(T, row0 + (i / ND) * 16, (i % ND) * 32, lane);
#pragma unroll
    for (int step = 0; step < N; step++) {
        if (step + PF < N)
            a[(step + PF) % (PF + 1)] = lds_operand_tr_swz<D>(T, row0 + ((step + PF) / ND) * 16, ((step + PF) % ND) * 32, lane);
        __builtin_amdgcn_sched_barrier(0);
        acc[step % ND] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[step % (PF + 1)], b[step / ND], acc[step % ND], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        hook(step);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// The same two GEMM loops with the LDS byte addresses of the lane's operands passed in (one per head-dimension block:
// the swizzle makes them differ per lane, not by a constant) plus an immediate: a kernel that has no registers left to
// unroll its tile loop over the LDS buffers keeps these addresses in registers and flips them between the buffers with one
// XOR each per tile, instead of rebuilding every address from pointer + swizzle before each read.
typedef __attribute__((address_space(3))) const bf16x8 *lds_bf16x8_ptr;
typedef __attribute__((address_space(3))) i16x4 *lds_i16x4_ptr;

template <int D>
__device__ __forceinline__ void lds_gemm_pair_at(const unsigned (&addr)[D / 16], int imm_a, int imm_b,
                                                 const bf16x8 (&ba)[D / 16], const bf16x8 (&bb)[D / 16], f32x16 &ra, f32x16 &rb) {
    constexpr int NK = D / 16, PF = 2;
    bf16x8 xa[PF + 1], xb[PF + 1];
#pragma unroll
    for (int i = 0; i < PF; i++) {
        xa[i] = *(lds_bf16x8_ptr)(uintptr_t)(addr[i] + imm_a);
        xb[i] = *(lds_bf16x8_ptr)(uintptr_t)(addr[i] + imm_b);
    }
#pragma unroll
    for (int kb = 0; kb < NK; kb++) {
        if (kb + PF < NK) {
            xa[(kb + PF) % (PF + 1)] = *(lds_bf16x8_ptr)(uintptr_t)(addr[kb + PF] + imm_a);
            xb[(kb + PF) % (PF + 1)] = *(lds_bf16x8_ptr)(uintptr_t)(addr[kb + PF] + imm_b);
        }
        __builtin_amdgcn_sched_barrier(0);
        ra = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[kb % (PF + 1)], ba[kb], ra, 0, 0, 0);
        rb = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xb[kb % (PF + 1)], bb[kb], rb, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// addr[j][h]: byte address of the lane's transpose-read element for head-dimension block j, rows +0 (h = 0) / +8 (h = 1)
template <int D, int NKB>
__device__ __forceinline__ void lds_tr_gemm_at(const unsigned (&addr)[D / 32][2], int imm, const bf16x8 (&b)[NKB], f32x16 (&acc)[D / 32]) {
    constexpr int ND = D / 32, N = NKB * ND, PF = 3;
    auto operand = [&](int i) {
        const int off = imm + (i / ND) * 16 * D * 2;
        union {
            struct { i16x4 a, b; } s;
            bf16x8 v;
        } u;
        u.s.a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr)(uintptr_t)(addr[i % ND][0] + off));
        u.s.b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr)(uintptr_t)(addr[i % ND][1] + off));
        return u.v;
    };
    bf16x8 a[PF + 1];
#pragma unroll
    for (int i = 0; i < PF && i < N; i++) a[i] = operand(i);
#pragma unroll
    for (int step = 0; step < N; step++) {
        if (step + PF < N) a[(step + PF) % (PF + 1)] = operand(step + PF);
        __builtin_amdgcn_sched_barrier(0);
        acc[step % ND] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[step % (PF + 1)], b[step / ND], acc[step % ND], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// Epilogue helper: a wave turns its 32 x D result tile, held in MFMA accumulator layout (lane (row l32, half hh),
// accumulator (db, 4 g + e) -> column 32 db + 8 g + 4 hh + e), into row-major order through a wave-private LDS area, so
// that global memory is written (and, for accumulators, read) in runs of whole rows instead of 8-16 bytes per row
// and instruction.  emit(row, col, v) receives 4 consecutive columns of one row; 32 / (D / 4) ... rows per step.
template <int D>
struct WaveStage {
    static constexpr int ROW_BYTES = D * 4 + 16;          // padded rows: the 128-bit column writes hit every bank once
    static constexpr int BYTES = 32 * ROW_BYTES + 128;    // + one float per row (per-row factor of the caller)
};

// Wave-uniform values pinned in scalar registers: kernel arguments used inside the epilogue loops are otherwise
// re-read from the argument segment in every iteration (a scalar load and a wait each time).
__device__ __forceinline__ int uniform32(int x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ long long uniform64(long long x) {
    const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)x), hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(x >> 32));
    return (long long)(((unsigned long long)hi << 32) | lo);
}

template <int D, class Emit>
__device__ __forceinline__ void wave_tile_rowmajor(unsigned char *stage, int lane, const f32x16 (&acc)[D / 32], float mul,
                                                   Emit emit) {
    const int l32 = lane & 31, hh = lane >> 5;
#pragma unroll
    for (int db = 0; db < D / 32; db++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            f32x4 v;
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = acc[db][4 * g + e] * mul;
            *(f32x4 *)(stage + l32 * WaveStage<D>::ROW_BYTES + (32 * db + 8 * g + 4 * hh) * 4) = v;
        }
    constexpr int LPR = D / 4;                // lanes per row
#pragma unroll
    for (int it = 0; it < 32 * LPR / 64; it++) {
        const int idx = it * 64 + lane, row = idx / LPR, c4 = idx % LPR;
        emit(row, 4 * c4, *(const f32x4 *)(stage + row * WaveStage<D>::ROW_BYTES + c4 * 16));
    }
}

// lds_gemm_chain / lds_tr_gemm for a wave that owns KW 32-key halves (dK/dV kernel) or KW 32-row blocks (forward): every operand
// read from LDS feeds one MFMA per half (b[k], r[k] / acc[k] belong to half k); hook(step) follows the MFMAs of operand `step`.
template <int D, int KW, class Hook = NoHook>
__device__ __forceinline__ void lds_gemm_chain_kw(const __bf16 *row, int sw, const bf16x8 (&b)[KW][D / 16], f32x16 (&r)[KW],
                                                  Hook hook = Hook()) {
    constexpr int NK = D / 16, PF = 2;
    bf16x8 x[PF + 1];
#pragma unroll
    for (int i = 0; i < PF; i++) x[i] = *(const bf16x8 *)(row + (((2 * i) ^ sw) << 3));
#pragma unroll
    for (int kb = 0; kb < NK; kb++) {
        if (kb + PF < NK) x[(kb + PF) % (PF + 1)] = *(const bf16x8 *)(row + (((2 * (kb + PF)) ^ sw) << 3));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k = 0; k < KW; k++) r[k] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x[kb % (PF + 1)], b[k][kb], r[k], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        hook(kb);
        __builtin_amdgcn_sched_barrier(0);
    }
}
template <int D, int NKB, int KW, class Hook = NoHook>
__device__ __forceinline__ void lds_tr_gemm_kw(const __bf16 *T, int row0, int lane, const bf16x8 (&b)[KW][NKB],
                                               f32x16 (&acc)[KW][D / 32], Hook hook = Hook()) {
    constexpr int ND = D / 32, N = NKB * ND, PF = 3;
    bf16x8 a[PF + 1];
#pragma unroll
    for (int i = 0; i < PF && i < N; i++) a[i] = lds_operand_tr_swz<D>(T, row0 + (i / ND) * 16, (i % ND) * 32, lane);
#pragma unroll
    for (int step = 0; step < N; step++) {
        if (step + PF < N)
            a[(step + PF) % (PF + 1)] = lds_operand_tr_swz<D>(T, row0 + ((step + PF) / ND) * 16, ((step + PF) % ND) * 32, lane);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k = 0; k < KW; k++)
            acc[k][step % ND] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[step % (PF + 1)], b[k][step / ND], acc[k][step % ND], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        hook(step);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// keys per K / V tile of the forward and dQ kernels
template <int D, int RB = 1>
struct FwdTile {
    static constexpr int BN = (D == 64 && RB == 1) ? 128 : 64;   // two row blocks per wave: S^T of 128 keys would be 128 registers
};

// ------------------------------------------------------------------------------ forward, bf16
// RB = 32-row blocks per wave.  With two (head dim 64) every K / V operand read from LDS feeds two MFMAs and a tile of
// 64 keys serves 512 query rows: half the LDS reads and half the tile transfers per MFMA.
template <int D, int RB>
__global__ __launch_bounds__(512) void fwd_bf16_kernel(const FwdParams p) {
    constexpr int NW = 8, BM = 32 * RB * NW;   // 8 waves (two per SIMD) share every K / V tile
    constexpr int BN = FwdTile<D, RB>::BN, NB = BN / 32;   // keys per tile: 32 KB (16 KB with two row blocks per wave)
    constexpr int CPR = D / 8;   // 16-byte chunks per row
    constexpr int RPI = 64 / CPR;            // rows filled by one wave-wide 16-byte-per-lane LDS-direct load (1 KB)
    constexpr int NI = BN / (RPI * NW);       // such loads per wave, per tensor and per tile
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];   // two {K tile, V tile} buffers,
    constexpr int TILE = BN * D;             // rows unpadded, 16-byte chunks XOR-swizzled (lds_swz)
    constexpr int BUF_ELEMS = 2 * TILE;

    const int tid = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool causal = p.flags & LTR_CAUSAL;

    // block -> (batch, kv head, q head of the group, q tile).  Consecutive block ids go to
    // the 8 XCDs round-robin; all q tiles / q heads of one (batch, kv head) run on one XCD and
    // next to each other in time, so the blocks that are resident together stream the same K/V
    // through that XCD's L2.  Late (heavier under a causal mask) q tiles first.
    int idx = blockIdx.x, pair, rest;
    const int P = p.B * p.Hkv;
    if ((P & 7) == 0) {
        int xcd = idx & 7, j = idx >> 3, nr = p.n_slots * p.n_rep;
        pair = (j / nr) * 8 + xcd;
        rest = j % nr;
    } else {
        pair = idx % P;
        rest = idx / P;
    }
    const int rep = rest % p.n_rep, slot = rest / p.n_rep;
    const int b = pair / p.Hkv, hkv = pair % p.Hkv, h = hkv * p.n_rep + rep;
    // A slot is one q tile (late, heavier tiles first) or, when the host paired them, a late tile and its early
    // counterpart: under a causal mask every block then has the same amount of work.
    const bool paired = p.n_slots != p.n_qtiles;
    // every other block (of an XCD) takes the early tile first: the blocks of a round then change tiles at different times
    const bool two = paired && slot < p.n_qtiles - 1 - slot, early_first = two && ((blockIdx.x >> 3) & 1);
#pragma nounroll
    for (int part = 0; part < 2; part++) {
    const int qt = (part == 0) != early_first ? p.n_qtiles - 1 - slot : slot;
    if (part == 1 && !two) break;
    if (part == 1) __syncthreads();   // the first tile's epilogue used the LDS buffers as staging areas
    // the lane index is made opaque per tile: everything derived from it (LDS addresses of the tile loop ...) is then
    // computed inside the tile's own scope instead of being hoisted out of this loop and kept alive across the epilogue
    int lane_of_part = threadIdx.x & 63;
    asm volatile("" : "+v"(lane_of_part));
    const int lane = lane_of_part, l32 = lane & 31, hh = lane >> 5;

    const int row0 = qt * BM;
    int my_row[RB], my_pos[RB];   // row block rb of wave w: rows row0 + 32 * (RB * w + rb) ..
    bool row_ok[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        my_row[rb] = row0 + (w * RB + rb) * 32 + l32;
        row_ok[rb] = my_row[rb] < p.Sq;
        my_pos[rb] = q_position(my_row[rb], p.q_split, p.q_pos0[0], p.q_pos0[1]);
    }
    int blk_lo, blk_hi, w_lo, w_hi;
    q_pos_range(row0, min(row0 + BM, p.Sq) - 1, p.q_split, p.q_pos0[0], p.q_pos0[1], blk_lo, blk_hi);
    {
        int wr0 = row0 + w * 32 * RB, wr1 = min(wr0 + 32 * RB, p.Sq) - 1;
        if (wr1 >= wr0) q_pos_range(wr0, wr1, p.q_split, p.q_pos0[0], p.q_pos0[1], w_lo, w_hi);
        else { w_lo = 0x7fffffff; w_hi = -0x7fffffff; }  // wave has no valid row
    }

    // Q operand (B of S^T = K Q^T): lane (query l32, half hh) holds d = 16*kb + 8*hh .. +7
    bf16x8 qreg[RB][D / 16];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        const __bf16 *qp = (const __bf16 *)p.q + b * p.qs[0] + (long long)my_row[rb] * p.qs[1] + h * p.qs[2];
#pragma unroll
        for (int kb = 0; kb < D / 16; kb++) {
            uint4 x = make_uint4(0, 0, 0, 0);
            if (row_ok[rb]) x = *(const uint4 *)(qp + kb * 16 + 8 * hh);
            qreg[rb][kb] = as_bf16x8(x);
        }
        // fused RoPE prologue: q arrives un-rotated and is rotated here, in the registers that hold it as the MFMA operand,
        // by the angles of the row's global position; the rotated row can be stored for the backward
        if ((p.flags & LTR_ROPE_Q) && row_ok[rb]) {
            const float *fr = p.rope + (long long)(my_pos[rb] - p.rope_pos0) * D + 8 * hh;
            __bf16 *qr = p.q_rot ? (__bf16 *)p.q_rot + b * p.qrs[0] + (long long)my_row[rb] * p.qrs[1] + h * p.qrs[2] + 8 * hh : nullptr;
#pragma unroll
            for (int kb = 0; kb < D / 16; kb++) {
                qreg[rb][kb] = rope_rotate8(qreg[rb][kb], *(const f32x4 *)(fr + 16 * kb), *(const f32x4 *)(fr + 16 * kb + 4));
                if (qr) *(bf16x8 *)(qr + 16 * kb) = qreg[rb][kb];
            }
        }
    }

    f32x16 zero16;
#pragma unroll
    for (int r = 0; r < 16; r++) zero16[r] = 0.f;
    f32x16 oacc[RB][D / 32];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int i = 0; i < D / 32; i++) oacc[rb][i] = zero16;
    // Online softmax state of this lane's query row.  mc is the reference point of the exponent (exp2 domain:
    // m * scale * log2(e)).  It does not follow the running max: P = exp2(s*c2 - mc) keeps its relative precision
    // whatever mc is, l and O accumulate in fp32 and LSE = mc*ln2 + log(l) is unaffected, so mc only has to keep
    // the row sum inside [TINY, BIG] where neither overflow nor flushed small terms matter.  That is checked on
    // the row sum of each tile (two compares), and the row max is only computed on the rare tile that fails the
    // check: the common tile has no max reduction and no rescale of the O accumulator.
    float mc[RB], l_run[RB];  // l_run: this lane's partial row sum (its half of the keys of every tile)
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        mc[rb] = 0.f;
        l_run[rb] = 0.f;
    }
    const float c2 = p.scale * LTR_LOG2E;
    constexpr float BIG = 1.152921504606846976e18f, TINY = 8.673617379884035472e-19f;   // 2^60, 2^-60

    // tile iterator over (chunk, key tile)
    // The fields of the chunk being loaded live in scalar registers and are re-read from the argument
    // table only when the chunk changes (a scalar load per tile would share the LDS wait counter).
    int c = -1, t = 0, nt = 0;
    int ld_sk = 0, ld_pos0 = 0;
    const __bf16 *ld_kb = nullptr, *ld_vb = nullptr;
    auto settle = [&]() {
        while (c < p.n_chunks && t >= nt) {
            c++;
            t = 0;
            if (c < p.n_chunks) {
                ld_sk = p.chunk[c].sk;
                ld_pos0 = p.chunk[c].pos0;
                ld_kb = (const __bf16 *)p.chunk[c].k + b * p.ks[0] + hkv * p.ks[2];
                ld_vb = (const __bf16 *)p.chunk[c].v + b * p.vs[0] + hkv * p.vs[2];
                const int nvis = causal ? max(0, min(ld_sk, blk_hi - ld_pos0 + 1)) : ld_sk;
                nt = (nvis + BN - 1) / BN;
            }
        }
    };
    settle();

    // Tiles go from global memory straight into LDS (global_load_lds, 16 bytes per lane, no staging
    // registers): wave w fills rows RPI*(NI*w + i) .. of the tile with its i-th load, lane l the chunk
    // position l % CPR of row l / CPR, fetching the logical chunk that the swizzle places there.  Rows past
    // the end of a chunk are fetched from its last row; their keys are masked.
    const int st_row = lane / CPR, st_pc = lane % CPR;
    int nx_sk = 0, nx_pos0 = 0, nx_key0 = 0;   // the tile in flight: becomes the tile computed next
    // transfer j of the tile in flight (ti, into buffer buf): j < NI are this wave's K rows, the rest its V rows
    auto gload_one = [&](int j, int ti, int buf) {
        const int i = j % NI;
        const unsigned dst = lds_address(smem) + buf * BUF_ELEMS * 2 + (j / NI) * TILE * 2 + RPI * (NI * w + i) * D * 2;
        const int row = RPI * (NI * w + i) + st_row;
        const int key = min(ti * BN + row, ld_sk - 1);
        const int chunk = st_pc ^ lds_swz<D>(row);
        const __bf16 *src = j < NI ? ld_kb + (long long)(key * (int)p.ks[1] + chunk * 8)
                                   : ld_vb + (long long)(key * (int)p.vs[1] + chunk * 8);
        global_to_lds_b128(src, dst);
    };
    auto gload_begin = [&](int ti) {   // scalar state of the tile whose transfers are issued next
        nx_sk = ld_sk;
        nx_pos0 = ld_pos0;
        nx_key0 = ti * BN;
    };

    // Double-buffered LDS, one barrier per tile: tile t+1 streams into the other buffer (whose readers all
    // passed the previous barrier) while tile t is computed; the barrier also waits for those loads.
    bool have = c < p.n_chunks;
    // Merging an empty partial result leaves (O, LSE) as they are: a block that sees no key of this launch's chunks (the
    // early rows of a causal ring step) skips the read-modify-write of its rows altogether.
    if (!have && (p.flags & LTR_MERGE)) continue;
    if (have) {
        gload_begin(t);
#pragma unroll
        for (int j = 0; j < 2 * NI; j++) gload_one(j, t, 0);
    }
    tile_barrier();
    // One tile; the loop below is unrolled over the two LDS buffers so that every LDS address is a loop-invariant
    // per-lane register plus an immediate offset (no address arithmetic between the MFMAs).
    auto tile_step = [&](auto par_tag) {
        constexpr int par = decltype(par_tag)::value;
        const int sk = nx_sk, pos0 = nx_pos0, key0 = nx_key0;
        const __bf16 *Ks = (const __bf16 *)smem + par * BUF_ELEMS, *Vs = Ks + TILE;
        t++;
        settle();
        const bool have_next = c < p.n_chunks;
        // All transfers of the next tile are issued here, right after the barrier: the memory pipe takes them
        // at 64 bytes per clock and a wave waits at the issue port meanwhile; issued between MFMAs instead
        // (measured) the same waits cost more, because they then stall waves that are feeding the matrix pipe.
        if (have_next) {
            gload_begin(t);
#pragma unroll
            for (int j = 0; j < 2 * NI; j++) gload_one(j, t, par ^ 1);
        }

        // A wave whose 32 rows all precede the tile's first key (upper part of a diagonal tile, rows past the end) has
        // nothing to add: it only takes part in the transfers and the barrier.
        if (!causal || pos0 + key0 <= w_hi) {
        // S^T of the two 32-key blocks of the tile.  The wave raises its priority while it issues MFMAs: the
        // other wave of the SIMD then fills the gaps with its softmax arithmetic instead of delaying them.
        __builtin_amdgcn_s_setprio(1);
        f32x16 s[NB][RB];
        if constexpr (RB == 1) {
#pragma unroll
            for (int nb = 0; nb < NB; nb += 2) {
                s[nb][0] = zero16;
                s[nb + 1][0] = zero16;
                lds_gemm_pair<D>(Ks + (nb * 32 + l32) * D, lds_swz<D>(nb * 32 + l32) ^ hh, Ks + (nb * 32 + 32 + l32) * D,
                                 lds_swz<D>(nb * 32 + 32 + l32) ^ hh, qreg[0], qreg[0], s[nb][0], s[nb + 1][0]);
            }
        } else {
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
#pragma unroll
                for (int rb = 0; rb < RB; rb++) s[nb][rb] = zero16;
                lds_gemm_chain_kw<D, RB>(Ks + (nb * 32 + l32) * D, lds_swz<D>(nb * 32 + l32) ^ hh, qreg, s[nb]);
            }
        }
        __builtin_amdgcn_s_setprio(0);
        // mask fix-up (tail of the chunk, diagonal tiles): wave-uniform branch touching S only
        const bool need_mask = (key0 + BN > sk) || (causal && (pos0 + key0 + BN - 1 > w_lo));
        if (need_mask) {
#pragma unroll
            for (int rb = 0; rb < RB; rb++)
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int key = key0 + nb * 32 + 8 * (r / 4) + 4 * hh + (r % 4);
                        const bool vis = key < sk && (!causal || pos0 + key <= my_pos[rb]);
                        s[nb][rb][r] = vis ? s[nb][rb][r] : -INFINITY;
                    }
        }
        // t = s*c2 - reference (exp2 domain), P = exp2(t) rounded to bf16, row sum of the rounded P (what PV uses)
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
#pragma unroll
                for (int r = 0; r < 16; r++) s[nb][rb][r] = s[nb][rb][r] * c2 - mc[rb];
        PackedTile pt[RB][NB];
        bf16x2 ones;
        ones[0] = (__bf16)1.0f;
        ones[1] = (__bf16)1.0f;
        float l_tile[RB];
        auto exponentials = [&](int rb) {
            l_tile[rb] = 0.f;
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    bf16x2 pr;
                    pr[0] = (__bf16)__builtin_amdgcn_exp2f(s[nb][rb][2 * j]);
                    pr[1] = (__bf16)__builtin_amdgcn_exp2f(s[nb][rb][2 * j + 1]);
                    l_tile[rb] = __builtin_amdgcn_fdot2_f32_bf16(pr, ones, l_tile[rb], false);
                    pt[rb][nb].u[j] = __builtin_bit_cast(unsigned, pr);
                }
        };
        bool out_of_range = false;
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            exponentials(rb);
            // in range: the tile's sum did not overflow and the row has a healthy sum by now (a lane sees half of the
            // row's keys, so its partial sum can lag behind the row's: that only costs a visit of the branch below)
            out_of_range = out_of_range || !(l_tile[rb] < BIG) || !(l_run[rb] + l_tile[rb] >= TINY);
        }
        if (__builtin_amdgcn_ballot_w64(out_of_range) != 0) {
#pragma unroll
            for (int rb = 0; rb < RB; rb++) {
                float mx = -INFINITY;
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
#pragma unroll
                    for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[nb][rb][r]);
                mx = xhalf_max(mx);                       // row max of t over the tile (-inf: no visible key)
                const float l_row = xhalf_sum(l_run[rb]), lt_row = xhalf_sum(l_tile[rb]);   // whole-row sums: both halves agree
                const bool row_bad = !(lt_row < BIG) || !(l_row + lt_row >= TINY);
                // New reference for a row that is out of range: the larger of the tile's max and the magnitude of the
                // history (log2 of its sum), so that neither overflows after the move; with a history never below -126, so
                // that the factor applied to it stays finite.  Rows that are in range, and rows that have seen no key at
                // all, keep theirs.
                const float hist = l_row > 0.f ? __log2f(l_row) : -INFINITY;
                const float target = fmaxf(mx, hist);
                const float shift = (row_bad && target > -INFINITY) ? (l_row > 0.f ? fmaxf(target, -126.f) : target) : 0.f;
                const float alpha = l_row > 0.f ? __builtin_amdgcn_exp2f(-shift) : 1.f;
                l_run[rb] *= alpha;
#pragma unroll
                for (int i = 0; i < D / 32; i++)
#pragma unroll
                    for (int r = 0; r < 16; r++) oacc[rb][i][r] *= alpha;
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
#pragma unroll
                    for (int r = 0; r < 16; r++) s[nb][rb][r] -= shift;
                mc[rb] += shift;
                exponentials(rb);
            }
        }
#pragma unroll
        for (int rb = 0; rb < RB; rb++) l_run[rb] += l_tile[rb];
        __builtin_amdgcn_s_setprio(1);
        if constexpr (RB == 1) {
            bf16x8 pb[2 * NB];
#pragma unroll
            for (int kb = 0; kb < 2 * NB; kb++) pb[kb] = operand_of(pt[0][kb >> 1], kb & 1);
            lds_tr_gemm<D, 2 * NB>(Vs, 0, lane, pb, oacc[0]);   // 16 keys per MFMA
        } else {
            bf16x8 pb[RB][2 * NB];
#pragma unroll
            for (int rb = 0; rb < RB; rb++)
#pragma unroll
                for (int kb = 0; kb < 2 * NB; kb++) pb[rb][kb] = operand_of(pt[rb][kb >> 1], kb & 1);
            lds_tr_gemm_kw<D, 2 * NB, RB>(Vs, 0, lane, pb, oacc);   // 16 keys per MFMA, one V operand read for both row blocks
        }
        __builtin_amdgcn_s_setprio(0);
        }
        tile_barrier();
        have = have_next;
    };
    while (have) {
        tile_step(std::integral_constant<int, 0>{});
        if (!have) break;
        tile_step(std::integral_constant<int, 1>{});
    }

    // epilogue: normalise, optional merge with the partial result already in (o, lse); one row block after the other
    // through the same staging area
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
    const float l_tot = xhalf_sum(l_run[rb]);
    float lse_new = (l_tot > 0.f) ? mc[rb] * LTR_LN2 + logf(l_tot) : -INFINITY;
    float w_cur = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
    float w_old = 0.f;
    float *lse_p = p.lse + ((long long)b * p.Hq + h) * p.Sq + my_row[rb];
    if ((p.flags & LTR_MERGE) && row_ok[rb]) {
        const float lse_old = *lse_p;
        const float mxl = fmaxf(lse_old, lse_new);
        if (mxl == -INFINITY) {
            w_cur = 0.f;
        } else {
            const float e_old = expf(lse_old - mxl), e_new = expf(lse_new - mxl);
            const float tot = e_old + e_new;
            w_old = e_old / tot;
            w_cur *= e_new / tot;
            lse_new = mxl + logf(tot);
        }
    }
    if (row_ok[rb] && hh == 0) *lse_p = lse_new;
    // O through the wave's LDS staging area (the tiles are no longer read: the last barrier is behind us)
    unsigned char *stage = smem + w * WaveStage<D>::BYTES;
    float *row_w_old = (float *)(stage + 32 * WaveStage<D>::ROW_BYTES);
    if (hh == 0) row_w_old[l32] = w_old;
    constexpr int LPR = D / 4, ROWS_PER_IT = 64 / LPR;      // see wave_tile_rowmajor
    const int Sq_u = uniform32(p.Sq), wave_row0 = uniform32(row0 + (w * RB + rb) * 32);
    const bool merge = uniform32(p.flags & LTR_MERGE) != 0, o_f32 = uniform32(p.o_f32) != 0;
    const long long os1 = uniform64(p.os[1]);
    const long long off0 = uniform64(b * p.os[0] + h * p.os[2]) + (wave_row0 + lane / LPR) * os1 + 4 * (lane % LPR);
    // merging: all reads of the earlier partial result first (independent loads in flight together), then the writes
    constexpr int NIT = 32 / ROWS_PER_IT;
    f32x4 old[NIT];
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        old[it] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (merge && wave_row0 + it * ROWS_PER_IT + lane / LPR < Sq_u) {
            if (o_f32) {
                old[it] = *(const f32x4 *)((const float *)p.o + off0 + it * ROWS_PER_IT * os1);
            } else {
                const bf16x4 x = *(const bf16x4 *)((const __bf16 *)p.o + off0 + it * ROWS_PER_IT * os1);
#pragma unroll
                for (int e = 0; e < 4; e++) old[it][e] = (float)x[e];
            }
        }
    }
    int it = 0;
    if (o_f32) {
        float *op = (float *)p.o + off0;
        wave_tile_rowmajor<D>(stage, lane, oacc[rb], w_cur, [&](int row, int, f32x4 val) {
            if (wave_row0 + row < Sq_u) {
                if (merge) {
                    const float wo = row_w_old[row];
#pragma unroll
                    for (int e = 0; e < 4; e++) val[e] += old[it][e] * wo;
                }
                *(f32x4 *)op = val;
            }
            op += ROWS_PER_IT * os1;
            it++;
        });
    } else {
        __bf16 *op = (__bf16 *)p.o + off0;
        wave_tile_rowmajor<D>(stage, lane, oacc[rb], w_cur, [&](int row, int, f32x4 val) {
            if (wave_row0 + row < Sq_u) {
                if (merge) {
                    const float wo = row_w_old[row];
#pragma unroll
                    for (int e = 0; e < 4; e++) val[e] += old[it][e] * wo;
                }
                bf16x4 ob;
#pragma unroll
                for (int e = 0; e < 4; e++) ob[e] = (__bf16)val[e];
                *(bf16x4 *)op = ob;
            }
            op += ROWS_PER_IT * os1;
            it++;
        });
    }
    }   // row block
    }   // part
}

// ------------------------------------------------------------------------------ forward, fp32
// One lane per query row, 64 rows per block, K/V tiles of 32 keys broadcast from LDS.
template <int D>
__global__ __launch_bounds__(64) void fwd_f32_kernel(const FwdParams p) {
    constexpr int BN = 32;
    __shared__ __attribute__((aligned(16))) float Ks[BN * D];
    __shared__ __attribute__((aligned(16))) float Vs[BN * D];
    const int tid = threadIdx.x;
    const bool causal = p.flags & LTR_CAUSAL;
    int idx = blockIdx.x;
    const int qt = p.n_qtiles - 1 - idx / (p.B * p.Hq);
    const int bh = idx % (p.B * p.Hq);
    const int b = bh / p.Hq, h = bh % p.Hq, hkv = h / p.n_rep;
    const int row0 = qt * 64, my_row = row0 + tid;
    const bool row_ok = my_row < p.Sq;
    const int my_pos = q_position(my_row, p.q_split, p.q_pos0[0], p.q_pos0[1]);
    int blk_lo, blk_hi;
    q_pos_range(row0, min(row0 + 64, p.Sq) - 1, p.q_split, p.q_pos0[0], p.q_pos0[1], blk_lo, blk_hi);

    float q[D], o[D];
    {
        const float *qp = (const float *)p.q + b * p.qs[0] + (long long)my_row * p.qs[1] + h * p.qs[2];
#pragma unroll
        for (int d = 0; d < D; d++) {
            q[d] = row_ok ? qp[d] : 0.f;
            o[d] = 0.f;
        }
    }
    float m_run = -INFINITY, l_run = 0.f;
    for (int c = 0; c < p.n_chunks; c++) {
        const int sk = p.chunk[c].sk, pos0 = p.chunk[c].pos0;
        const int nvis = causal ? max(0, min(sk, blk_hi - pos0 + 1)) : sk;
        const float *kp = (const float *)p.chunk[c].k + b * p.ks[0] + hkv * p.ks[2];
        const float *vp = (const float *)p.chunk[c].v + b * p.vs[0] + hkv * p.vs[2];
        for (int key0 = 0; key0 < nvis; key0 += BN) {
            __syncthreads();
            for (int i = tid; i < BN * D / 4; i += 64) {
                int key = key0 + i / (D / 4), dc = i % (D / 4);
                f32x4 kv = {0.f, 0.f, 0.f, 0.f}, vv = {0.f, 0.f, 0.f, 0.f};
                if (key < sk) {
                    kv = *(const f32x4 *)(kp + (long long)key * p.ks[1] + dc * 4);
                    vv = *(const f32x4 *)(vp + (long long)key * p.vs[1] + dc * 4);
                }
                *(f32x4 *)(Ks + i * 4) = kv;
                *(f32x4 *)(Vs + i * 4) = vv;
            }
            __syncthreads();
            float s[BN];
            float mx = -INFINITY;
#pragma unroll
            for (int j = 0; j < BN; j++) {
                float acc = 0.f;
#pragma unroll
                for (int d = 0; d < D; d++) acc = fmaf(q[d], Ks[j * D + d], acc);
                acc *= p.scale;
                const int key = key0 + j;
                const bool vis = key < sk && (!causal || pos0 + key <= my_pos);
                s[j] = vis ? acc : -INFINITY;
                mx = fmaxf(mx, s[j]);
            }
            const float m_new = fmaxf(m_run, mx);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = expf(m_run - m_use);
            l_run *= alpha;
#pragma unroll
            for (int d = 0; d < D; d++) o[d] *= alpha;
#pragma unroll
            for (int j = 0; j < BN; j++) {
                const float pj = expf(s[j] - m_use);
                l_run += pj;
#pragma unroll
                for (int d = 0; d < D; d++) o[d] = fmaf(pj, Vs[j * D + d], o[d]);
            }
            m_run = m_new;
        }
    }
    if (!row_ok) return;
    float lse_new = (l_run > 0.f) ? m_run + logf(l_run) : -INFINITY;
    float w_cur = (l_run > 0.f) ? 1.f / l_run : 0.f, w_old = 0.f;
    float *lse_p = p.lse + ((long long)b * p.Hq + h) * p.Sq + my_row;
    if (p.flags & LTR_MERGE) {
        const float lse_old = *lse_p;
        const float mxl = fmaxf(lse_old, lse_new);
        if (mxl == -INFINITY) {
            w_cur = 0.f;
        } else {
            const float e_old = expf(lse_old - mxl), e_new = expf(lse_new - mxl);
            const float tot = e_old + e_new;
            w_old = e_old / tot;
            w_cur *= e_new / tot;
            lse_new = mxl + logf(tot);
        }
    }
    *lse_p = lse_new;
    float *op = (float *)p.o + b * p.os[0] + (long long)my_row * p.os[1] + h * p.os[2];
#pragma unroll
    for (int d = 0; d < D; d++) {
        float val = o[d] * w_cur;
        if (p.flags & LTR_MERGE) val += op[d] * w_old;
        op[d] = val;
    }
}

// ------------------------------------------------------------------------------ forward, fp32 on the matrix pipe
// v_mfma_f32_32x32x2_f32 (lane l, i = l % 32, h = l / 32: A[i][h], B[h][i], C as for the bf16 shape): fp32 operands and
// fp32 accumulation, so the 1e-4 cases run on the matrix pipe at full precision.  A block has 4 waves; a wave owns 32 query
// rows (a lane = one query, as in the bf16 kernel) and one of KS interleaved shares of the keys: the RG = 4 / KS waves with
// different rows share every K / V tile, the KS waves with the same rows take the sub-tiles ks, ks + KS, ... of 32 keys and
// their partial (m, l, O) are merged at the end.  KS > 1 is for launches with too few query rows to fill the device (the
// reference's acceptance shapes).  Both contractions pick their own order of the contraction index so that no operand moves:
//   S^T = K Q^T   step 4g + j contracts d = 8g + 4h + j: the K operand of four steps is one 128-bit LDS read, Q stays in
//                 registers in that order;
//   O^T += V^T P^T  step r contracts the key of accumulator register r (8 (r / 4) + 4h + r % 4): P^T is used where it is.
// K / V tiles of 32 * KS keys go global -> LDS directly, double buffered, 16-byte chunks XOR-swizzled (f32_swz) so that the
// 128-bit K reads (16 rows, same chunk) and the 32-bit V reads (one row per half-wave, rows 4 apart) touch every bank once.
__device__ __forceinline__ int f32_swz(int row) {   // bits 2 and 3 of the row swapped: rows 4 apart land 32 banks apart
    return (row & 3) | (((row >> 2) & 1) << 3) | (((row >> 3) & 1) << 2);
}

template <int D, int KS>
struct F32Mfma {
    static constexpr int NW = 4, RG = NW / KS;          // waves; row groups of 32 rows
    static constexpr int BM = 32 * RG, BN = 32 * KS;    // rows per block, keys per step
    static constexpr int TILE = BN * D;                 // floats per K (or V) tile
    static constexpr int BUF_BYTES = 2 * TILE * 4;      // {K tile, V tile}
    static constexpr int ML_OFF = 0, ML_BYTES = NW * 64 * 4;                        // per wave: m[32], l[32]
    static constexpr int PART_OFF = ML_BYTES, PART_BYTES = (D / 32) * 16 * 64 * 4;  // one wave's O^T accumulators, lane-major
    static constexpr int MERGE_BYTES = PART_OFF + (KS - 1) * RG * PART_BYTES;
    static constexpr int STAGE_OFF = MERGE_BYTES;       // row-major staging of the RG writing waves, after the merge area
    static constexpr int EPI_BYTES = STAGE_OFF + RG * WaveStage<D>::BYTES;
    static constexpr int LDS = 2 * BUF_BYTES > EPI_BYTES ? 2 * BUF_BYTES : EPI_BYTES;
    static_assert(LDS <= 160 * 1024, "LDS of one CU");
};

template <int D, int KS>
__global__ __launch_bounds__(256) void fwd_f32_mfma_kernel(const FwdParams p) {
    using L = F32Mfma<D, KS>;
    constexpr int NW = L::NW, RG = L::RG, BM = L::BM, BN = L::BN, TILE = L::TILE;
    constexpr int CPR = D / 4;               // 16-byte chunks per row
    constexpr int RPI = 64 / CPR;            // rows filled by one wave-wide LDS-direct load (1 KB)
    constexpr int NI = BN / (RPI * NW);      // such loads per wave, per tensor and per step
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, hh = lane >> 5;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rg = w / KS, ks = w % KS;
    const bool causal = p.flags & LTR_CAUSAL;
    int idx = blockIdx.x;
    const int qt = p.n_qtiles - 1 - idx / (p.B * p.Hq);     // late (heavier under a causal mask) q tiles first
    const int bh = idx % (p.B * p.Hq);
    const int b = bh / p.Hq, h = bh % p.Hq, hkv = h / p.n_rep;
    const int row0 = qt * BM, my_row = row0 + rg * 32 + l32;
    const bool row_ok = my_row < p.Sq;
    const int my_pos = q_position(my_row, p.q_split, p.q_pos0[0], p.q_pos0[1]);
    int blk_lo, blk_hi, w_lo, w_hi;
    q_pos_range(row0, min(row0 + BM, p.Sq) - 1, p.q_split, p.q_pos0[0], p.q_pos0[1], blk_lo, blk_hi);
    {
        const int wr0 = row0 + rg * 32, wr1 = min(wr0 + 32, p.Sq) - 1;
        if (wr1 >= wr0) q_pos_range(wr0, wr1, p.q_split, p.q_pos0[0], p.q_pos0[1], w_lo, w_hi);
        else { w_lo = 0x7fffffff; w_hi = -0x7fffffff; }   // wave has no valid row
    }

    // Q operand: qreg[4g + j] = Q[row][8g + 4h + j]
    float qreg[D / 2];
    {
        const float *qp = (const float *)p.q + b * p.qs[0] + (long long)min(my_row, p.Sq - 1) * p.qs[1] + h * p.qs[2];
#pragma unroll
        for (int g = 0; g < D / 8; g++) {
            f32x4 x = *(const f32x4 *)(qp + 8 * g + 4 * hh);
            if (!row_ok) x = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 4; j++) qreg[4 * g + j] = x[j];
        }
    }
    f32x16 oacc[D / 32];
#pragma unroll
    for (int i = 0; i < D / 32; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[i][r] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;   // exp2 domain; l_run: this lane's half of the keys
    const float c2 = p.scale * LTR_LOG2E;

    // step iterator over (chunk, BN keys); chunk fields live in scalar registers (see the bf16 kernel)
    int c = -1, t = 0, nt = 0;
    int ld_sk = 0, ld_pos0 = 0;
    const float *ld_kb = nullptr, *ld_vb = nullptr;
    auto settle = [&]() {
        while (c < p.n_chunks && t >= nt) {
            c++;
            t = 0;
            if (c < p.n_chunks) {
                ld_sk = p.chunk[c].sk;
                ld_pos0 = p.chunk[c].pos0;
                ld_kb = (const float *)p.chunk[c].k + b * p.ks[0] + hkv * p.ks[2];
                ld_vb = (const float *)p.chunk[c].v + b * p.vs[0] + hkv * p.vs[2];
                const int nvis = causal ? max(0, min(ld_sk, blk_hi - ld_pos0 + 1)) : ld_sk;
                nt = (nvis + BN - 1) / BN;
            }
        }
    };
    settle();
    const int st_row = lane / CPR, st_pc = lane % CPR;
    int nx_sk = 0, nx_pos0 = 0, nx_key0 = 0;
    auto gload = [&](int ti, int buf) {
        nx_sk = ld_sk;
        nx_pos0 = ld_pos0;
        nx_key0 = ti * BN;
        const unsigned Kd = lds_address(smem) + buf * L::BUF_BYTES, Vd = Kd + TILE * 4;
#pragma unroll
        for (int i = 0; i < NI; i++) {
            const int row = RPI * (NI * w + i) + st_row;
            const int key = min(ti * BN + row, ld_sk - 1);       // rows past the end repeat the last row; they are masked
            const int chunk = st_pc ^ f32_swz(row);
            global_to_lds_b128(ld_kb + ((long long)key * p.ks[1] + chunk * 4), Kd + RPI * (NI * w + i) * D * 4);
            global_to_lds_b128(ld_vb + ((long long)key * p.vs[1] + chunk * 4), Vd + RPI * (NI * w + i) * D * 4);
        }
    };
    bool have = c < p.n_chunks;
    if (!have && (p.flags & LTR_MERGE)) return;   // merging an empty partial result changes nothing (block-uniform)
    if (have) gload(t, 0);
    tile_barrier();
    int par = 0;
    while (have) {
        const int sk = nx_sk, pos0 = nx_pos0, key0 = nx_key0 + 32 * ks;   // this wave's 32 keys of the step
        const float *Ks = (const float *)(smem + par * L::BUF_BYTES) + 32 * ks * D, *Vs = Ks + TILE;
        t++;
        settle();
        const bool have_next = c < p.n_chunks;
        if (have_next) gload(t, par ^ 1);
        // nothing to add: the sub-tile starts past the chunk's end, or every row of the wave precedes its first key
        if (key0 < sk && (!causal || pos0 + key0 <= w_hi)) {
            f32x16 s;
#pragma unroll
            for (int r = 0; r < 16; r++) s[r] = 0.f;
            const float *krow = Ks + l32 * D;
            const int ksw = f32_swz(l32);
#pragma unroll
            for (int g = 0; g < D / 8; g++) {
                const f32x4 kx = *(const f32x4 *)(krow + (((2 * g + hh) ^ ksw) << 2));
#pragma unroll
                for (int j = 0; j < 4; j++) s = __builtin_amdgcn_mfma_f32_32x32x2f32(kx[j], qreg[4 * g + j], s, 0, 0, 0);
            }
            const bool need_mask = (key0 + 32 > sk) || (causal && (pos0 + key0 + 31 > w_lo));
            float mx = -INFINITY;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float tv = s[r] * c2;
                if (need_mask) {
                    const int key = key0 + 8 * (r / 4) + 4 * hh + (r % 4);
                    const bool vis = key < sk && (!causal || pos0 + key <= my_pos);
                    tv = vis ? tv : -INFINITY;
                }
                s[r] = tv;
                mx = fmaxf(mx, tv);
            }
            mx = xhalf_max(mx);                                   // row max over the 32 keys (both halves agree)
            const float m_new = fmaxf(m_run, mx);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);   // m_run = -inf: 0 (nothing accumulated yet)
            float l_tile = 0.f;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                s[r] = __builtin_amdgcn_exp2f(s[r] - m_use);
                l_tile += s[r];
            }
            l_run = l_run * alpha + l_tile;
            m_run = m_new;
#pragma unroll
            for (int i = 0; i < D / 32; i++)
#pragma unroll
                for (int r = 0; r < 16; r++) oacc[i][r] *= alpha;
            // O^T += V^T P^T: step r contracts key 8 (r / 4) + 4h + r % 4; lane (d = 32 db + l32, h) reads V[key][d]
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int vrow = 8 * (r / 4) + 4 * hh + (r % 4);
                const float *vr = Vs + vrow * D + (l32 & 3);
                const int vsw = f32_swz(vrow);
#pragma unroll
                for (int db = 0; db < D / 32; db++) {
                    const float vx = vr[((8 * db + (l32 >> 2)) ^ vsw) << 2];
                    oacc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(vx, s[r], oacc[db], 0, 0, 0);
                }
            }
        }
        tile_barrier();
        par ^= 1;
        have = have_next;
    }

    // merge of the KS partial results of a row group (the tile buffers are no longer read: the last barrier is behind us)
    float l_tot = xhalf_sum(l_run);
    if constexpr (KS > 1) {
        float *ml = (float *)(smem + L::ML_OFF);
        if (hh == 0) {
            ml[w * 64 + l32] = m_run;
            ml[w * 64 + 32 + l32] = l_tot;
        }
        __syncthreads();
        float m_all = -INFINITY;
#pragma unroll
        for (int k2 = 0; k2 < KS; k2++) m_all = fmaxf(m_all, ml[(rg * KS + k2) * 64 + l32]);
        const float m_ref = m_all == -INFINITY ? 0.f : m_all;
        float l_sum = 0.f;
#pragma unroll
        for (int k2 = 0; k2 < KS; k2++)
            l_sum += ml[(rg * KS + k2) * 64 + 32 + l32] * __builtin_amdgcn_exp2f(ml[(rg * KS + k2) * 64 + l32] - m_ref);
        const float f_own = __builtin_amdgcn_exp2f(m_run - m_ref);
        float *part = (float *)(smem + L::PART_OFF);
        if (ks > 0) {
            float *mine = part + (size_t)(rg * (KS - 1) + ks - 1) * (L::PART_BYTES / 4);
#pragma unroll
            for (int i = 0; i < D / 32; i++)
#pragma unroll
                for (int r4 = 0; r4 < 4; r4++) {
                    f32x4 x;
#pragma unroll
                    for (int e = 0; e < 4; e++) x[e] = oacc[i][4 * r4 + e] * f_own;
                    *(f32x4 *)(mine + ((i * 4 + r4) * 64 + lane) * 4) = x;
                }
        }
        __syncthreads();
        if (ks == 0) {
#pragma unroll
            for (int i = 0; i < D / 32; i++)
#pragma unroll
                for (int r = 0; r < 16; r++) oacc[i][r] *= f_own;
            for (int k2 = 1; k2 < KS; k2++) {
                const float *other = part + (size_t)(rg * (KS - 1) + k2 - 1) * (L::PART_BYTES / 4);
#pragma unroll
                for (int i = 0; i < D / 32; i++)
#pragma unroll
                    for (int r4 = 0; r4 < 4; r4++) {
                        const f32x4 x = *(const f32x4 *)(other + ((i * 4 + r4) * 64 + lane) * 4);
#pragma unroll
                        for (int e = 0; e < 4; e++) oacc[i][4 * r4 + e] += x[e];
                    }
            }
        }
        m_run = m_all;
        l_tot = l_sum;
        if (ks > 0) return;    // no barrier follows
    }

    // epilogue of the wave that holds the row group's result: normalise, optional merge with (o, lse), whole rows out
    float lse_new = (l_tot > 0.f) ? m_run * LTR_LN2 + logf(l_tot) : -INFINITY;
    float w_cur = (l_tot > 0.f) ? 1.f / l_tot : 0.f, w_old = 0.f;
    float *lse_p = p.lse + ((long long)b * p.Hq + h) * p.Sq + my_row;
    if ((p.flags & LTR_MERGE) && row_ok) {
        const float lse_old = *lse_p;
        const float mxl = fmaxf(lse_old, lse_new);
        if (mxl == -INFINITY) {
            w_cur = 0.f;
        } else {
            const float e_old = expf(lse_old - mxl), e_new = expf(lse_new - mxl);
            const float tot = e_old + e_new;
            w_old = e_old / tot;
            w_cur *= e_new / tot;
            lse_new = mxl + logf(tot);
        }
    }
    if (row_ok && hh == 0) *lse_p = lse_new;
    unsigned char *stage = smem + L::STAGE_OFF + rg * WaveStage<D>::BYTES;
    float *row_w_old = (float *)(stage + 32 * WaveStage<D>::ROW_BYTES);
    if (hh == 0) row_w_old[l32] = w_old;
    constexpr int LPR = D / 4, ROWS_PER_IT = 64 / LPR;
    const int wave_row0 = row0 + rg * 32;
    const bool merge = (p.flags & LTR_MERGE) != 0;
    float *op = (float *)p.o + b * p.os[0] + h * p.os[2] + (long long)(wave_row0 + lane / LPR) * p.os[1] + 4 * (lane % LPR);
    const long long os1 = p.os[1];
    const int Sq = p.Sq;
    wave_tile_rowmajor<D>(stage, lane, oacc, w_cur, [&](int row, int, f32x4 val) {
        if (wave_row0 + row < Sq) {
            if (merge) {
                const f32x4 old = *(const f32x4 *)op;
                const float wo = row_w_old[row];
#pragma unroll
                for (int e = 0; e < 4; e++) val[e] += old[e] * wo;
            }
            *(f32x4 *)op = val;
        }
        op += ROWS_PER_IT * os1;
    });
}

// ------------------------------------------------------------------------------ delta
// 16 lanes per (b, h, row); each lane covers D/16 contiguous elements.
__global__ __launch_bounds__(256) void delta_kernel(const DeltaParams p) {
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long rowid = gid >> 4;
    const int sub = gid & 15;
    const long long nrows = (long long)p.B * p.Hq * p.Sq;
    float acc = 0.f;
    if (rowid < nrows) {
        const int i = rowid % p.Sq;
        const int h = (rowid / p.Sq) % p.Hq;
        const int b = rowid / ((long long)p.Sq * p.Hq);
        const long long oo = b * p.os[0] + (long long)i * p.os[1] + h * p.os[2];
        const long long od = b * p.dos[0] + (long long)i * p.dos[1] + h * p.dos[2];
        const int per = p.D / 16;
        for (int e = 0; e < per; e++) {
            const int d = sub * per + e;
            const float ov = p.o_f32 ? ((const float *)p.o)[oo + d] : (float)((const __bf16 *)p.o)[oo + d];
            const float dv = p.do_f32 ? ((const float *)p.d_o)[od + d] : (float)((const __bf16 *)p.d_o)[od + d];
            acc = fmaf(ov, dv, acc);
        }
    }
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 16);
    if (rowid < nrows && sub == 0) p.delta[rowid] = acc;
}

__global__ __launch_bounds__(256) void cast_kernel(const float *src, __bf16 *dst, long long n) {
    long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i + 3 < n) {
        f32x4 x = *(const f32x4 *)(src + i);
        bf16x4 y;
#pragma unroll
        for (int e = 0; e < 4; e++) y[e] = (__bf16)x[e];
        *(bf16x4 *)(dst + i) = y;
    } else {
        for (; i < n; i++) dst[i] = (__bf16)src[i];
    }
}

// ------------------------------------------------------------------------------ backward, bf16
// Two kernels, no atomics, bitwise reproducible:
//   bwd_dkdv_kernel  a block owns 128 keys of one kv head and runs 8 waves, two per SIMD: for each of
//                    the four 32-key slices one "P wave" (S = Q K^T, P, dV^T += dO^T P; K operand in
//                    registers) and one "dS wave" (dP = dO V^T, dS = P*(dP - DELTA), dK^T += Q^T dS;
//                    V operand in registers).  The P wave hands P (bf16, accumulator layout) to its
//                    partner through a 2 KB LDS slot; the dS wave runs one tile behind, so one block
//                    barrier per tile is enough.  The block loops over the query heads of the GQA
//                    group and over 64-row Q / dO tiles in triple-buffered LDS; dK^T and dV^T stay
//                    in registers for the whole loop.
//   bwd_dq_kernel    a block owns 256 query rows of one query head (32 per wave; Q and dO
//                    operands in registers), loops over 64-key K/V tiles like the forward;
//                    dQ^T accumulates in registers.
// LDS of bwd_dkdv_kernel (dynamic): three buffers of {Q tile, dO tile, -LSE/scale, -DELTA, row positions}, the P slots,
// the tile lists.
template <int D, int KW>
struct BwdLds {
    static constexpr int BN = 128 * KW; // keys per block, 32 * KW per wave pair
    static constexpr int BM = 64;       // query rows per tile (two 32-row MFMA sub-tiles)
    static constexpr int NT = 512;      // threads per block
    static constexpr int TILE = BM * D;                                  // elements; rows unpadded, chunks swizzled
    static constexpr int BUF_BYTES = 2 * TILE * 2 + 3 * BM * 4;          // Q, dO, -LSE/scale, -DELTA, row positions (masked tiles)
    static constexpr int P_SLOT = 64 * 32;                               // one lane = 16 bf16 = 32 bytes
    static constexpr int NBUF = 3;                                       // tile t (P waves), t-1 (dS waves), t+1 (in flight)
    static constexpr int P_OFF = NBUF * BUF_BYTES;
    static constexpr int MAX_QTILES = 4096;                              // Sq <= 262144 per launch
    static constexpr int LIST_OFF = P_OFF + 4 * 4 * KW * P_SLOT;         // 4 slices x 2 parities x 2 sub-tiles x KW halves of P slots
    static constexpr int TOTAL = LIST_OFF + 2 * MAX_QTILES * 2 + 16;     // two tile lists (ushort) + counts
    static_assert(TOTAL >= 8 * WaveStage<D>::BYTES, "the epilogue's staging areas reuse this memory");
    static_assert(TOTAL <= 160 * 1024, "LDS of one CU");
};

// Masked tiles: the visibility of (row, key) is kpos <= qpos[row], with the rows' positions staged in LDS beside LSE and
// DELTA (INT_MIN for a row past the end; INT_MAX - 1 for every row when there is no causal mask) and kpos = INT_MAX for
// a key past the end of its chunk: one compare and one select per element, whatever the position map of the rows is.
constexpr int BWD_QPOS_NONE = (int)0x80000000, BWD_QPOS_ALL = 0x7ffffffe, BWD_KPOS_NONE = 0x7fffffff;

// P wave, accumulator registers 2j and 2j+1 of a 32x32 sub-tile: sm = S - LSE / scale (the accumulator started at
// -LSE / scale), P = exp2(sm * c2) -> one packed bf16 pair in accumulator layout; qpos = positions of the sub-tile's 16
// rows in accumulator-register order
template <bool MASK>
__device__ __forceinline__ unsigned bwd_p_pair(const f32x16 &sm, int j, float c2, int kpos, const int (&qpos)[16]) {
    float p0 = __builtin_amdgcn_exp2f(sm[2 * j] * c2), p1 = __builtin_amdgcn_exp2f(sm[2 * j + 1] * c2);
    if (MASK) {
        p0 = kpos <= qpos[2 * j] ? p0 : 0.f;
        p1 = kpos <= qpos[2 * j + 1] ? p1 : 0.f;
    }
    return pack2_bf16(p0, p1);
}

// dS wave, the same pair: dS = P * (dP - DELTA), pu = packed P pair from the partner's LDS slot (masked entries
// are 0), dpm = dP - DELTA (the accumulator started at -DELTA)
__device__ __forceinline__ unsigned bwd_ds_pair(unsigned pu, const f32x16 &dpm, int j) {
    const float p0 = __uint_as_float(pu << 16), p1 = __uint_as_float(pu & 0xffff0000u);
    return pack2_bf16(p0 * dpm[2 * j], p1 * dpm[2 * j + 1]);
}

template <int D, int KW>
__global__ __launch_bounds__(512) void bwd_dkdv_kernel(const BwdParams p) {
    using L = BwdLds<D, KW>;   // KW = 32-key halves per wave
    constexpr int BN = L::BN, BM = L::BM;
    constexpr int CPR = D / 8;
    constexpr int RPI = 64 / CPR;        // rows filled by one wave-wide LDS-direct load (1 KB)
    constexpr int NI = BM / (RPI * 8);   // such loads per wave, per tensor and per tile
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int slice = w & 3;             // slice of 32 * KW keys; waves w and w+4 (same SIMD) are partners
    const bool p_role = w < 4;           // P wave (S, P, dV) or dS wave (dP, dS, dK)
    const int l32 = lane & 31, hh = lane >> 5;
    const bool causal = p.flags & LTR_CAUSAL;

    // block -> (batch, kv head, chunk, key tile); same XCD grouping as the forward
    int idx = blockIdx.x, pair, rest;
    const int P = p.B * p.Hkv;
    if ((P & 7) == 0) {
        int xcd = idx & 7, j = idx >> 3;
        pair = (j / p.tiles_total) * 8 + xcd;
        rest = j % p.tiles_total;
    } else {
        pair = idx % P;
        rest = idx / P;
    }
    const int b = pair / p.Hkv, hkv = pair % p.Hkv;
    int c = 0, kt = rest;
    for (; c < p.n_chunks; c++) {
        int n = (p.chunk[c].sk + BN - 1) / BN;
        if (kt < n) break;
        kt -= n;
    }
    if (c >= p.n_chunks) return;
    const int sk = p.chunk[c].sk, pos0 = p.chunk[c].pos0;
    const int key0 = kt * BN;
    int my_key[KW];   // this lane's keys in the S / dP / dK^T / dV^T tiles of the wave's two halves
    bool key_ok[KW];
#pragma unroll
    for (int k = 0; k < KW; k++) {
        my_key[k] = key0 + slice * 32 * KW + 32 * k + l32;
        key_ok[k] = my_key[k] < sk;
    }
    const int tile_kpos_lo = pos0 + key0;
    const int tile_kpos_hi = pos0 + min(key0 + BN, sk) - 1;
    const bool key_tail = key0 + BN > sk;
    if (causal) {   // no query of this launch sees the block (a later chunk of the ring): nothing to add, nothing to load
        int q_lo, q_hi;
        q_pos_range(0, (int)p.Sq - 1, p.q_split, p.q_pos0[0], p.q_pos0[1], q_lo, q_hi);
        if (q_hi < tile_kpos_lo) {
            for (int k = 0; k < KW; k++)
            if ((p.flags & LTR_DKDV_BF16) && key_ok[k]) {   // results, not accumulators: these keys get zeros
                __bf16 *gz = p_role ? (__bf16 *)p.chunk[c].dv + b * p.dvs[0] + (long long)my_key[k] * p.dvs[1] + hkv * p.dvs[2]
                                    : (__bf16 *)p.chunk[c].dk + b * p.dks[0] + (long long)my_key[k] * p.dks[1] + hkv * p.dks[2];
                for (int d = 8 * hh; d < D; d += 16) *(uint4 *)(gz + d) = make_uint4(0, 0, 0, 0);
            }
            return;
        }
    }

    // resident B operand: K rows for a P wave, V rows for a dS wave; lane (key l32, half hh) holds
    // d = 16*kb + 8*hh .. +7
    bf16x8 kvreg[KW][D / 16];
    {
        const __bf16 *base = p_role ? (const __bf16 *)p.chunk[c].k + b * p.ks[0] + hkv * p.ks[2]
                                    : (const __bf16 *)p.chunk[c].v + b * p.vs[0] + hkv * p.vs[2];
        const long long rs = p_role ? p.ks[1] : p.vs[1];
#pragma unroll
        for (int k = 0; k < KW; k++) {
            const int ksafe = min(my_key[k], sk - 1);
#pragma unroll
            for (int kb = 0; kb < D / 16; kb++) {
                uint4 x = *(const uint4 *)(base + (long long)ksafe * rs + kb * 16 + 8 * hh);
                if (!key_ok[k]) x = make_uint4(0, 0, 0, 0);
                kvreg[k][kb] = as_bf16x8(x);
            }
        }
    }

    f32x16 zero16;
#pragma unroll
    for (int r = 0; r < 16; r++) zero16[r] = 0.f;
    f32x16 acc[KW][D / 32];              // dV^T (P wave) or dK^T (dS wave) of the two halves
#pragma unroll
    for (int k = 0; k < KW; k++)
#pragma unroll
        for (int i = 0; i < D / 32; i++) acc[k][i] = zero16;
    const float c2 = p.scale * LTR_LOG2E;

    // A tile's class depends on its rows only: 0 = no row sees any key of the block (skipped);
    // 1 = every (row, key) pair is visible; 2 = needs the mask (diagonal, tails).
    auto tile_class = [&](int qt) {
        const int row0 = qt * BM;
        const bool edge = key_tail || row0 + BM > p.Sq;
        if (!causal) return edge ? 2 : 1;
        int lo, hi;
        q_pos_range(row0, min(row0 + BM, p.Sq) - 1, p.q_split, p.q_pos0[0], p.q_pos0[1], lo, hi);
        if (hi < tile_kpos_lo) return 0;
        return (edge || tile_kpos_hi > lo) ? 2 : 1;
    };

    // The q tiles of each class are listed once per block (wave 0, ballot compaction: the order, and with it
    // the rounding of the accumulation, is fixed), so the main loops carry no classification arithmetic.
    unsigned short *const tlist = (unsigned short *)(smem + L::LIST_OFF);     // [2][MAX_QTILES]
    int *const tcount = (int *)(smem + L::LIST_OFF + 2 * L::MAX_QTILES * 2);
    if (w == 0) {
        int n1 = 0, n2 = 0;
        for (int base = 0; base < p.n_qtiles; base += 64) {
            const int qt = base + lane;
            const int cls = qt < p.n_qtiles ? tile_class(qt) : 0;
            const unsigned long long m1 = __builtin_amdgcn_ballot_w64(cls == 1), m2 = __builtin_amdgcn_ballot_w64(cls == 2);
            const unsigned long long below = (1ull << lane) - 1ull;
            if (cls == 1) tlist[n1 + __builtin_popcountll(m1 & below)] = (unsigned short)qt;
            if (cls == 2) tlist[L::MAX_QTILES + n2 + __builtin_popcountll(m2 & below)] = (unsigned short)qt;
            n1 += __builtin_popcountll(m1);
            n2 += __builtin_popcountll(m2);
        }
        if (lane == 0) {
            tcount[0] = n1;
            tcount[1] = n2;
        }
    }
    __syncthreads();

    const int st_row = lane / CPR, st_pc = lane % CPR;   // this lane's place inside a 1 KB LDS-direct load
    // Per-lane element offsets of this lane's pieces of a Q / dO tile (unmasked tiles: row and chunk do not depend on the
    // tile) and the bases of the current q head: a step then adds one scalar product per tensor instead of redoing the
    // 64-bit address arithmetic of (batch, head, row).
    unsigned offq[NI], offdo[NI];
#pragma unroll
    for (int i = 0; i < NI; i++) {
        const int row = RPI * (NI * w + i) + st_row;
        const int chunk = st_pc ^ lds_swz<D>(row);
        offq[i] = (unsigned)(row * (int)p.qs[1] + chunk * 8);
        offdo[i] = (unsigned)(row * (int)p.dos[1] + chunk * 8);
    }
    const __bf16 *qp_head = nullptr, *dop_head = nullptr;
    const float *sp_head = nullptr;   // LSE (wave 0) or DELTA - BM (wave 1) of the head's rows, indexed by row0 + tid
    auto set_head = [&](int rep) __attribute__((always_inline)) {
        const int h = hkv * p.n_rep + rep;
        qp_head = (const __bf16 *)p.q + b * p.qs[0] + h * p.qs[2];
        dop_head = (const __bf16 *)p.d_o + b * p.dos[0] + h * p.dos[2];
        const long long so = ((long long)b * p.Hq + h) * p.Sq;
        sp_head = w == 0 ? p.lse + so : p.delta + so - BM;
    };
    const float st_mul = tid < BM ? -1.f / p.scale : -1.f;  // threads 0..63 stage -LSE/scale, 64..127 stage -DELTA
    float sld = 0.f;      // raw LSE / DELTA value in flight; scaled when it is written to LDS
    bool sld_ok = true;
    int sld_row0 = 0;     // first row of the tile in flight
    unsigned *const pslot_base = (unsigned *)(smem + L::P_OFF) + slice * 4 * KW * (L::P_SLOT / 4);   // [parity][sub-tile][half]

    // two passes, each a loop of its own (unmasked tiles, then masked ones), so the accumulators
    // live in straight-line loop bodies and the unmasked pass carries no bounds checks at all
    auto run_pass = [&](auto mask_tag) {
        constexpr bool MASK = decltype(mask_tag)::value;
        constexpr int cls = MASK ? 2 : 1;
        const int cnt = __builtin_amdgcn_readfirstlane(tcount[cls - 1]);
        const unsigned short *const list = tlist + (cls - 1) * L::MAX_QTILES;
        int li_ = -1;                                 // index into the list
        // the list entry of the next call is read from LDS one call ahead, so its latency is never waited for
        unsigned short pre = list[0];
        auto advance = [&](int &rep, int &qt) {   // next tile of this class after (rep, qt); false when done
            if (++li_ >= cnt) {
                li_ = 0;
                if (++rep >= p.n_rep) return false;
                set_head(rep);
            }
            qt = __builtin_amdgcn_readfirstlane((int)pre);
            pre = list[li_ + 1 < cnt ? li_ + 1 : 0];
            return true;
        };
        // Q and dO tiles go from global memory straight into LDS (global_load_lds, 16 bytes per lane): wave w
        // fills rows RPI*(NI*w + i) .. of both tiles with its i-th pair of loads, lane l the chunk position
        // l % CPR of row l / CPR, fetching the logical chunk the swizzle places there.  Rows past the end of Q
        // repeat its last row (they are masked).  LSE and DELTA go through a register of threads 0..127.
        auto gload = [&](int rep, int qt, int buf) {
            const int row0 = qt * BM;
            sld_row0 = row0;
            const unsigned Qd = lds_address(smem) + buf * L::BUF_BYTES, dOd = Qd + L::TILE * 2;   // LDS byte addresses
            if (!MASK) {
                const unsigned tq = (unsigned)(row0 * (int)p.qs[1]), tdo = (unsigned)(row0 * (int)p.dos[1]);
#pragma unroll
                for (int i = 0; i < NI; i++) {
                    global_to_lds_b128(qp_head + (unsigned long long)(tq + offq[i]), Qd + RPI * (NI * w + i) * D * 2);
                    global_to_lds_b128(dop_head + (unsigned long long)(tdo + offdo[i]), dOd + RPI * (NI * w + i) * D * 2);
                }
            } else {
#pragma unroll
                for (int i = 0; i < NI; i++) {
                    const int row = RPI * (NI * w + i) + st_row;
                    const int grow = min(row0 + row, p.Sq - 1);
                    const int chunk = st_pc ^ lds_swz<D>(row);
                    global_to_lds_b128(qp_head + (long long)(grow * (int)p.qs[1] + chunk * 8), Qd + RPI * (NI * w + i) * D * 2);
                    global_to_lds_b128(dop_head + (long long)(grow * (int)p.dos[1] + chunk * 8), dOd + RPI * (NI * w + i) * D * 2);
                }
            }
            if (tid < 2 * BM) {
                const float *sp = sp_head + row0;
                if (!MASK) {
                    sld = sp[tid];
                } else {
                    const int r = tid < BM ? tid : tid - BM;
                    sld_ok = row0 + r < p.Sq;
                    sld = sp[sld_ok ? tid : (tid < BM ? 0 : BM)];
                }
            }
        };
        auto lds_store = [&](int buf) {   // the LSE / DELTA values fetched by gload
            float *st = (float *)(smem + buf * L::BUF_BYTES) + L::TILE;   // after the two bf16 tiles
            if (tid < 2 * BM) {
                float x = sld * st_mul;
                // rows past the end: -LSE/scale = -inf makes P = 0 (they are masked as well)
                if (MASK) x = sld_ok ? x : (tid < BM ? -INFINITY : 0.f);
                st[tid] = x;
            } else if (MASK && tid < 3 * BM) {   // positions of the tile's rows (third wave)
                const int row = sld_row0 + tid - 2 * BM;
                ((int *)st)[tid] = row >= p.Sq ? BWD_QPOS_NONE
                                   : causal ? q_position(row, p.q_split, p.q_pos0[0], p.q_pos0[1]) : BWD_QPOS_ALL;
            }
        };

        int kpos[KW];
#pragma unroll
        for (int k = 0; k < KW; k++) kpos[k] = key_ok[k] ? pos0 + my_key[k] : BWD_KPOS_NONE;
        if (cnt == 0) return;
        int rep = 0, qt = 0;
        set_head(0);
        advance(rep, qt);
        __syncthreads();   // the previous pass has finished reading LDS
        gload(rep, qt, 0);
        lds_store(0);
        tile_barrier();
        // One LDS barrier per 64-row tile.  In step t the P wave does all its work on tile t (S of both
        // sub-tiles, P -> slots of parity t & 1, dV) and the dS wave all its work on tile t-1 (dP, dS with P
        // from the slots filled one step earlier, dK): inside a step the two waves of a SIMD are independent,
        // so one wave's softmax arithmetic runs under the other's MFMAs.  Slots of parity (t & 1) are
        // rewritten in step t+2, after the barrier that ends step t+1 in which they were read.  Tile t+1 is
        // fetched into registers at the start of step t and stored at its end into buffer (t+1) % 3, which
        // held tile t-2, last read in step t-1.  Both roles execute T + 1 barriers.
        auto put_slot = [&](unsigned *slot, const PackedTile &t) {
            // two 16-byte halves per lane, each half contiguous over the lanes (no bank conflicts)
            *(uint4 *)(slot + lane * 4) = make_uint4(t.u[0], t.u[1], t.u[2], t.u[3]);
            *(uint4 *)(slot + 256 + lane * 4) = make_uint4(t.u[4], t.u[5], t.u[6], t.u[7]);
        };
        int par = 0;
        // In the pass over unmasked tiles both loops are unrolled over the three Q / dO buffers (buf is a compile-time
        // constant inside a step), so that LDS addresses are loop-invariant per-lane registers plus immediate offsets;
        // the pass over masked tiles (few steps, more live registers) keeps one loop body with buf in a register.
        if (p_role) {
            bool more = true;
            auto p_step = [&](auto buf_tag) {
                const int buf = buf_tag;
                more = advance(rep, qt);
                const int nbuf = buf == L::NBUF - 1 ? 0 : buf + 1;
                if (more) gload(rep, qt, nbuf);
                const __bf16 *Qs = (const __bf16 *)(smem + buf * L::BUF_BYTES);
                const __bf16 *dOs = Qs + L::TILE;
                const float *st_s = (const float *)(dOs + L::TILE);   // -LSE/scale of the tile's rows
                unsigned *slots = pslot_base + par * 2 * KW * (L::P_SLOT / 4);
                // Accumulator register r of a sub-tile <-> tile row 8*(r/4) + 4*hh + r%4: both S accumulators start at
                // -LSE/scale of their rows.  Order of the step: S of sub-tile a; S of sub-tile b with the
                // exponentials of a issued under its MFMAs; first half of dV (rows of a) with the exponentials of b
                // under its MFMAs; second half of dV.
                f32x16 sa[KW], sb[KW];
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const f32x4 la = *(const f32x4 *)(st_s + 8 * g + 4 * hh), lb = *(const f32x4 *)(st_s + 32 + 8 * g + 4 * hh);
#pragma unroll
                    for (int k = 0; k < KW; k++)
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            sa[k][4 * g + e] = la[e];
                            sb[k][4 * g + e] = lb[e];
                        }
                }
                int qa[16], qb[16];   // positions of the rows (masked tiles only)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int *st_q = (const int *)st_s + 2 * BM;
                    const i32x4 xa = MASK ? *(const i32x4 *)(st_q + 8 * g + 4 * hh) : i32x4{0, 0, 0, 0};
                    const i32x4 xb = MASK ? *(const i32x4 *)(st_q + 32 + 8 * g + 4 * hh) : i32x4{0, 0, 0, 0};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        qa[4 * g + e] = xa[e];
                        qb[4 * g + e] = xb[e];
                    }
                }
                PackedTile ppa[KW], ppb[KW];
                constexpr int NK = D / 16, ND = D / 32;
                __builtin_amdgcn_s_setprio(1);
                // every Q / dO operand read from LDS feeds the MFMAs of both halves
                lds_gemm_chain_kw<D, KW>(Qs + l32 * D, lds_swz<D>(l32) ^ hh, kvreg, sa);
                lds_gemm_chain_kw<D, KW>(Qs + (32 + l32) * D, lds_swz<D>(32 + l32) ^ hh, kvreg, sb, [&](int kb) {
#pragma unroll
                    for (int k = 0; k < KW; k++)
#pragma unroll
                        for (int j = kb * (8 / NK); j < (kb + 1) * (8 / NK); j++) ppa[k].u[j] = bwd_p_pair<MASK>(sa[k], j, c2, kpos[k], qa);
                });
                bf16x8 pba[KW][2], pbb[KW][2];
#pragma unroll
                for (int k = 0; k < KW; k++) {
                    put_slot(slots + k * (L::P_SLOT / 4), ppa[k]);
                    pba[k][0] = operand_of(ppa[k], 0);
                    pba[k][1] = operand_of(ppa[k], 1);
                }
                lds_tr_gemm_kw<D, 2, KW>(dOs, 0, lane, pba, acc, [&](int step) {
#pragma unroll
                    for (int k = 0; k < KW; k++)
#pragma unroll
                        for (int j = step * (4 / ND); j < (step + 1) * (4 / ND); j++) ppb[k].u[j] = bwd_p_pair<MASK>(sb[k], j, c2, kpos[k], qb);
                });
#pragma unroll
                for (int k = 0; k < KW; k++) {
                    put_slot(slots + (KW + k) * (L::P_SLOT / 4), ppb[k]);
                    pbb[k][0] = operand_of(ppb[k], 0);
                    pbb[k][1] = operand_of(ppb[k], 1);
                }
                lds_tr_gemm_kw<D, 2, KW>(dOs, 32, lane, pbb, acc);
                __builtin_amdgcn_s_setprio(0);
                if (more) lds_store(nbuf);
                tile_barrier();
                par ^= 1;
            };
            static_assert(L::NBUF == 3, "unrolled over three buffers");
            if (MASK) {
                int buf = 0;
                while (more) {
                    p_step(buf);
                    buf = buf == L::NBUF - 1 ? 0 : buf + 1;
                }
            } else {
                for (;;) {
                    p_step(std::integral_constant<int, 0>{});
                    if (!more) break;
                    p_step(std::integral_constant<int, 1>{});
                    if (!more) break;
                    p_step(std::integral_constant<int, 2>{});
                    if (!more) break;
                }
            }
            tile_barrier();                        // step T: only the dS waves have work
        } else {
            bool more = advance(rep, qt);          // step 0: staging duties only
            if (more) gload(rep, qt, 1);
            tile_barrier();
            bool had_next = true;
            auto ds_step = [&](auto buf_tag) {
                const int buf = buf_tag;
                had_next = more;
                if (more) {
                    more = advance(rep, qt);
                    if (more) gload(rep, qt, buf + 2 >= L::NBUF ? buf + 2 - L::NBUF : buf + 2);
                }
                const __bf16 *Qs = (const __bf16 *)(smem + buf * L::BUF_BYTES);
                const __bf16 *dOs = Qs + L::TILE;
                const float *dlt_s = (const float *)(dOs + L::TILE) + BM;
                const unsigned *slots = pslot_base + par * 2 * KW * (L::P_SLOT / 4);
                // the dP accumulators start at -DELTA of their rows (register r <-> tile row 8*(r/4) + 4*hh + r%4);
                // same order as the P wave: dP of a; dP of b with dS of a under its MFMAs; first half of dK with dS of
                // b under its MFMAs; second half of dK
                f32x16 dpa[KW], dpb[KW];
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const f32x4 da = *(const f32x4 *)(dlt_s + 8 * g + 4 * hh), db4 = *(const f32x4 *)(dlt_s + 32 + 8 * g + 4 * hh);
#pragma unroll
                    for (int k = 0; k < KW; k++)
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            dpa[k][4 * g + e] = da[e];
                            dpb[k][4 * g + e] = db4[e];
                        }
                }
                PackedTile dsa[KW], dsb[KW];
                constexpr int NK = D / 16, ND = D / 32;
                __builtin_amdgcn_s_setprio(1);
                lds_gemm_chain_kw<D, KW>(dOs + l32 * D, lds_swz<D>(l32) ^ hh, kvreg, dpa);
                unsigned pua[KW][8], pub[KW][8];
#pragma unroll
                for (int k = 0; k < KW; k++) {
                    const unsigned *sl = slots + k * (L::P_SLOT / 4);
                    const uint4 pa0 = *(const uint4 *)(sl + lane * 4), pa1 = *(const uint4 *)(sl + 256 + lane * 4);
                    pua[k][0] = pa0.x; pua[k][1] = pa0.y; pua[k][2] = pa0.z; pua[k][3] = pa0.w;
                    pua[k][4] = pa1.x; pua[k][5] = pa1.y; pua[k][6] = pa1.z; pua[k][7] = pa1.w;
                }
                lds_gemm_chain_kw<D, KW>(dOs + (32 + l32) * D, lds_swz<D>(32 + l32) ^ hh, kvreg, dpb, [&](int kb) {
#pragma unroll
                    for (int k = 0; k < KW; k++)
#pragma unroll
                        for (int j = kb * (8 / NK); j < (kb + 1) * (8 / NK); j++) dsa[k].u[j] = bwd_ds_pair(pua[k][j], dpa[k], j);
                });
                bf16x8 dba[KW][2], dbb[KW][2];
#pragma unroll
                for (int k = 0; k < KW; k++) {
                    const unsigned *sl = slots + (KW + k) * (L::P_SLOT / 4);
                    const uint4 pb0 = *(const uint4 *)(sl + lane * 4), pb1 = *(const uint4 *)(sl + 256 + lane * 4);
                    pub[k][0] = pb0.x; pub[k][1] = pb0.y; pub[k][2] = pb0.z; pub[k][3] = pb0.w;
                    pub[k][4] = pb1.x; pub[k][5] = pb1.y; pub[k][6] = pb1.z; pub[k][7] = pb1.w;
                    dba[k][0] = operand_of(dsa[k], 0);
                    dba[k][1] = operand_of(dsa[k], 1);
                }
                lds_tr_gemm_kw<D, 2, KW>(Qs, 0, lane, dba, acc, [&](int step) {
#pragma unroll
                    for (int k = 0; k < KW; k++)
#pragma unroll
                        for (int j = step * (4 / ND); j < (step + 1) * (4 / ND); j++) dsb[k].u[j] = bwd_ds_pair(pub[k][j], dpb[k], j);
                });
#pragma unroll
                for (int k = 0; k < KW; k++) {
                    dbb[k][0] = operand_of(dsb[k], 0);
                    dbb[k][1] = operand_of(dsb[k], 1);
                }
                lds_tr_gemm_kw<D, 2, KW>(Qs, 32, lane, dbb, acc);
                __builtin_amdgcn_s_setprio(0);
                tile_barrier();
                par ^= 1;
            };
            if (MASK) {
                int buf = 0;
                while (had_next) {
                    ds_step(buf);
                    buf = buf == L::NBUF - 1 ? 0 : buf + 1;
                }
            } else {
                for (;;) {
                    ds_step(std::integral_constant<int, 0>{});
                    if (!had_next) break;
                    ds_step(std::integral_constant<int, 1>{});
                    if (!had_next) break;
                    ds_step(std::integral_constant<int, 2>{});
                    if (!had_next) break;
                }
            }
        }
    };
    run_pass(std::false_type{});
    run_pass(std::true_type{});

    // dV^T (P wave) / dK^T (dS wave) tile of the wave's 32 keys: added to the fp32 accumulators in whole rows, through the
    // wave's LDS staging area (every wave is past the last barrier: tiles, slots and lists are no longer read)
#pragma unroll
    for (int k = 0; k < KW; k++) {
        constexpr int LPR = D / 4, ROWS_PER_IT = 64 / LPR;      // see wave_tile_rowmajor
        const long long stride = uniform64(p_role ? p.dvs[1] : p.dks[1]);
        const int key_base = uniform32(key0 + slice * 32 * KW + 32 * k), sk_u = uniform32(sk);
        const long long goff = (p_role ? b * p.dvs[0] + hkv * p.dvs[2] : b * p.dks[0] + hkv * p.dks[2]) +
                               (key_base + lane / LPR) * stride + 4 * (lane % LPR);
        if (uniform32(p.flags & LTR_DKDV_BF16)) {   // every query that sees these keys was in this launch: store the result
            __bf16 *gb = (__bf16 *)(p_role ? p.chunk[c].dv : p.chunk[c].dk) + goff;
            wave_tile_rowmajor<D>(smem + w * WaveStage<D>::BYTES, lane, acc[k], p_role ? 1.f : p.scale, [&](int row, int, f32x4 val) {
                if (key_base + row < sk_u) {
                    bf16x4 y;
#pragma unroll
                    for (int e = 0; e < 4; e++) y[e] = (__bf16)val[e];
                    *(bf16x4 *)gb = y;
                }
                gb += ROWS_PER_IT * stride;
            });
            continue;
        }
        float *gp = (p_role ? p.chunk[c].dv : p.chunk[c].dk) + goff;
        // all reads of the accumulator first (independent loads in flight together), then the adds and the writes
        constexpr int NIT = 32 / ROWS_PER_IT;
        f32x4 old[NIT];
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            old[it] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (key_base + it * ROWS_PER_IT + lane / LPR < sk_u) old[it] = *(const f32x4 *)(gp + it * ROWS_PER_IT * stride);
        }
        int it = 0;
        wave_tile_rowmajor<D>(smem + w * WaveStage<D>::BYTES, lane, acc[k], p_role ? 1.f : p.scale, [&](int row, int, f32x4 val) {
            if (key_base + row < sk_u) {
#pragma unroll
                for (int e = 0; e < 4; e++) val[e] += old[it][e];
                *(f32x4 *)gp = val;
            }
            gp += ROWS_PER_IT * stride;
            it++;
        });
    }
}

// dQ: same block / wave / lane roles as the forward (a lane owns one query row), so LSE and DELTA are
// per-lane scalars.  S^T = K Q^T and dP^T = V dO^T with K, V tiles natural in LDS; dS^T leaves the
// registers as the B operand of dQ^T += K^T dS^T, whose A operand is the K tile read by transpose loads.
// lds_gemm_pair_at / lds_tr_gemm_at for a wave that owns RB 32-row blocks: every operand read from LDS feeds one MFMA per row
// block (ba[rb], bb[rb], ra[rb], rb_[rb] / b[rb], acc[rb] belong to row block rb).
template <int D, int RB>
__device__ __forceinline__ void lds_gemm_pair_at_rb(const unsigned (&addr)[D / 16], int imm_a, int imm_b, const bf16x8 (&ba)[RB][D / 16],
                                                    const bf16x8 (&bb)[RB][D / 16], f32x16 (&ra)[RB], f32x16 (&rb_)[RB]) {
    constexpr int NK = D / 16, PF = 2;
    bf16x8 xa[PF + 1], xb[PF + 1];
#pragma unroll
    for (int i = 0; i < PF; i++) {
        xa[i] = *(lds_bf16x8_ptr)(uintptr_t)(addr[i] + imm_a);
        xb[i] = *(lds_bf16x8_ptr)(uintptr_t)(addr[i] + imm_b);
    }
#pragma unroll
    for (int kb = 0; kb < NK; kb++) {
        if (kb + PF < NK) {
            xa[(kb + PF) % (PF + 1)] = *(lds_bf16x8_ptr)(uintptr_t)(addr[kb + PF] + imm_a);
            xb[(kb + PF) % (PF + 1)] = *(lds_bf16x8_ptr)(uintptr_t)(addr[kb + PF] + imm_b);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < RB; r++) {
            ra[r] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[kb % (PF + 1)], ba[r][kb], ra[r], 0, 0, 0);
            rb_[r] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xb[kb % (PF + 1)], bb[r][kb], rb_[r], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}
template <int D, int NKB, int RB>
__device__ __forceinline__ void lds_tr_gemm_at_rb(const unsigned (&addr)[D / 32][2], int imm, const bf16x8 (&b)[RB][NKB],
                                                  f32x16 (&acc)[RB][D / 32]) {
    constexpr int ND = D / 32, N = NKB * ND, PF = 3;
    auto operand = [&](int i) {
        const int off = imm + (i / ND) * 16 * D * 2;
        union {
            struct { i16x4 a, b; } s;
            bf16x8 v;
        } u;
        u.s.a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr)(uintptr_t)(addr[i % ND][0] + off));
        u.s.b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr)(uintptr_t)(addr[i % ND][1] + off));
        return u.v;
    };
    bf16x8 a[PF + 1];
#pragma unroll
    for (int i = 0; i < PF && i < N; i++) a[i] = operand(i);
#pragma unroll
    for (int step = 0; step < N; step++) {
        if (step + PF < N) a[(step + PF) % (PF + 1)] = operand(step + PF);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < RB; r++)
            acc[r][step % ND] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[step % (PF + 1)], b[r][step / ND], acc[r][step % ND], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
}

template <int D, int RB>   // RB = 32-row blocks per wave: a lane owns RB query rows, a block 256 * RB
__global__ __launch_bounds__(512) void bwd_dq_kernel(const BwdParams p) {
    constexpr int NW = 8, BM = 32 * RB * NW, BN = FwdTile<D>::BN;   // 8 waves (two per SIMD) share every K / V tile
    constexpr int CPR = D / 8;
    constexpr int RPI = 64 / CPR;            // rows filled by one wave-wide 16-byte-per-lane LDS-direct load (1 KB)
    constexpr int NI = BN / (RPI * NW);       // such loads per wave, per tensor and per tile
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];   // two {K tile, V tile} buffers,
    constexpr int TILE = BN * D;             // rows unpadded, 16-byte chunks XOR-swizzled (lds_swz)
    constexpr int BUF_ELEMS = 2 * TILE;

    const int tid = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool causal = p.flags & LTR_CAUSAL;

    int idx = blockIdx.x, pair, rest;
    const int P = p.B * p.Hkv;
    if ((P & 7) == 0) {
        int xcd = idx & 7, j = idx >> 3, nr = p.n_slots * p.n_rep;
        pair = (j / nr) * 8 + xcd;
        rest = j % nr;
    } else {
        pair = idx % P;
        rest = idx / P;
    }
    const int n_qt = (p.Sq + BM - 1) / BM;
    const int rep = rest % p.n_rep, slot = rest / p.n_rep;
    const int b = pair / p.Hkv, hkv = pair % p.Hkv, h = hkv * p.n_rep + rep;
    // one q tile per block (late tiles first) or a late tile and its early counterpart (see q_tile_slots)
    const bool paired = p.n_slots != n_qt;
    const bool two = paired && slot < n_qt - 1 - slot, early_first = two && ((blockIdx.x >> 3) & 1);   // as in the forward kernel
#pragma nounroll
    for (int part = 0; part < 2; part++) {
    const int qt = (part == 0) != early_first ? n_qt - 1 - slot : slot;
    if (part == 1 && !two) break;
    if (part == 1) __syncthreads();   // the first tile's epilogue used the LDS buffers as staging areas
    int lane_of_part = threadIdx.x & 63;   // opaque per tile, see the forward kernel
    asm volatile("" : "+v"(lane_of_part));
    const int lane = lane_of_part, l32 = lane & 31, hh = lane >> 5;

    const int row0 = qt * BM;
    int my_row[RB], my_pos[RB];
    bool row_ok[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        my_row[rb] = row0 + w * 32 * RB + 32 * rb + l32;
        row_ok[rb] = my_row[rb] < p.Sq;
        my_pos[rb] = q_position(my_row[rb], p.q_split, p.q_pos0[0], p.q_pos0[1]);
    }
    int blk_lo, blk_hi, w_lo, w_hi;
    q_pos_range(row0, min(row0 + BM, p.Sq) - 1, p.q_split, p.q_pos0[0], p.q_pos0[1], blk_lo, blk_hi);
    {
        int wr0 = row0 + w * 32 * RB, wr1 = min(wr0 + 32 * RB, p.Sq) - 1;
        if (wr1 >= wr0) q_pos_range(wr0, wr1, p.q_split, p.q_pos0[0], p.q_pos0[1], w_lo, w_hi);
        else { w_lo = -0x7fffffff; w_hi = -0x7fffffff; }  // wave has no valid row: everything masked
    }

    bf16x8 qreg[RB][D / 16], doreg[RB][D / 16];
    float lse2[RB], dlt[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        lse2[rb] = INFINITY;
        dlt[rb] = 0.f;
        const int rsafe = min(my_row[rb], p.Sq - 1);
        const __bf16 *qp = (const __bf16 *)p.q + b * p.qs[0] + (long long)rsafe * p.qs[1] + h * p.qs[2];
        const __bf16 *dop = (const __bf16 *)p.d_o + b * p.dos[0] + (long long)rsafe * p.dos[1] + h * p.dos[2];
#pragma unroll
        for (int kb = 0; kb < D / 16; kb++) {
            qreg[rb][kb] = as_bf16x8(*(const uint4 *)(qp + kb * 16 + 8 * hh));
            doreg[rb][kb] = as_bf16x8(*(const uint4 *)(dop + kb * 16 + 8 * hh));
        }
        if (p.flags & LTR_DELTA_FROM_O) {
            // DELTA = rowsum(dO * O) of this lane's row: its half of every 16-element block, then the other half's
            const __bf16 *op = (const __bf16 *)p.o + b * p.os_[0] + (long long)rsafe * p.os_[1] + h * p.os_[2];
            float part = 0.f;
#pragma unroll
            for (int kb = 0; kb < D / 16; kb++) {
                const bf16x8 ov = as_bf16x8(*(const uint4 *)(op + kb * 16 + 8 * hh));
#pragma unroll
                for (int e = 0; e < 8; e++) part += (float)ov[e] * (float)doreg[rb][kb][e];
            }
            dlt[rb] = xhalf_sum(part);
            if (row_ok[rb] && hh == 0) p.delta[((long long)b * p.Hq + h) * p.Sq + my_row[rb]] = dlt[rb];
        }
        if (row_ok[rb]) {
            // a row that saw no key has LSE = -inf: give it +inf like a row past the end, so that P = exp2(-inf) = 0
            // whatever S is (S = -inf after the mask fix-up would otherwise meet -(-inf))
            const float lse_row = p.lse[((long long)b * p.Hq + h) * p.Sq + my_row[rb]];
            lse2[rb] = lse_row == -INFINITY ? INFINITY : lse_row * LTR_LOG2E;
            if (!(p.flags & LTR_DELTA_FROM_O)) dlt[rb] = p.delta[((long long)b * p.Hq + h) * p.Sq + my_row[rb]];
        }
    }
    f32x16 zero16;
#pragma unroll
    for (int r = 0; r < 16; r++) zero16[r] = 0.f;
    f32x16 dqacc[RB][D / 32];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int i = 0; i < D / 32; i++) dqacc[rb][i] = zero16;
    // the dP^T accumulators start at -DELTA of the lane's row (the first MFMA of the chain takes this as its addend), so
    // dS = P * (dP - DELTA) needs no subtraction per element (one row block per wave only: with two the 16 registers per
    // row block are not there)
    constexpr bool DLT_INIT = RB == 1;
    f32x16 ndlt[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int r = 0; r < 16; r++) ndlt[rb][r] = DLT_INIT ? -dlt[rb] : 0.f;
    const float c2 = p.scale * LTR_LOG2E;

    // The fields of the chunk being loaded live in scalar registers and are re-read from the argument
    // table only when the chunk changes (a scalar load per tile would share the LDS wait counter).
    int c = -1, t = 0, nt = 0;
    int ld_sk = 0, ld_pos0 = 0;
    const __bf16 *ld_kb = nullptr, *ld_vb = nullptr;
    auto settle = [&]() {
        while (c < p.n_chunks && t >= nt) {
            c++;
            t = 0;
            if (c < p.n_chunks) {
                ld_sk = p.chunk[c].sk;
                ld_pos0 = p.chunk[c].pos0;
                ld_kb = (const __bf16 *)p.chunk[c].k + b * p.ks[0] + hkv * p.ks[2];
                ld_vb = (const __bf16 *)p.chunk[c].v + b * p.vs[0] + hkv * p.vs[2];
                const int nvis = causal ? max(0, min(ld_sk, blk_hi - ld_pos0 + 1)) : ld_sk;
                nt = (nvis + BN - 1) / BN;
            }
        }
    };
    settle();

    // Tiles go from global memory straight into LDS (see the forward kernel): wave w fills rows
    // RPI*(NI*w + i) .. with its i-th load; rows past the end of a chunk repeat its last row and are masked.
    const int st_row = lane / CPR, st_pc = lane % CPR;
    int nx_sk = 0, nx_pos0 = 0, nx_key0 = 0;   // the tile in flight: becomes the tile computed next
    auto gload = [&](int ti, int buf) {
        nx_sk = ld_sk;
        nx_pos0 = ld_pos0;
        nx_key0 = ti * BN;
        const unsigned Kd = lds_address(smem) + buf * BUF_ELEMS * 2, Vd = Kd + TILE * 2;   // LDS byte addresses
#pragma unroll
        for (int i = 0; i < NI; i++) {
            const int row = RPI * (NI * w + i) + st_row;
            const int key = min(ti * BN + row, ld_sk - 1);
            const int chunk = st_pc ^ lds_swz<D>(row);
            global_to_lds_b128(ld_kb + (long long)(key * (int)p.ks[1] + chunk * 8), Kd + RPI * (NI * w + i) * D * 2);
            global_to_lds_b128(ld_vb + (long long)(key * (int)p.vs[1] + chunk * 8), Vd + RPI * (NI * w + i) * D * 2);
        }
    };

    bool have = c < p.n_chunks;
    // a block that sees no key of this launch's chunks adds nothing to an fp32 dQ accumulator: no read-modify-write
    if (!have && !(p.flags & LTR_DQ_BF16)) continue;
    if (have) gload(t, 0);
    tile_barrier();
    // LDS byte addresses of this lane's operands in the K tile of the current buffer (the V tile and the other 32-key
    // blocks are immediates away): kept in registers and flipped to the other buffer with one XOR each per tile
    static_assert((BUF_ELEMS * 2 & (BUF_ELEMS * 2 - 1)) == 0, "buffer size must be a power of two for the XOR flip");
    unsigned pa[D / 16], ta[D / 32][2];
    {
        const unsigned lds0 = lds_address(smem);   // the only LDS object of the kernel: aligned far beyond the buffer size
        const int sw = lds_swz<D>(l32) ^ hh;        // rows l32 + 32 n share the swizzle word of row l32
#pragma unroll
        for (int kb = 0; kb < D / 16; kb++) pa[kb] = lds0 + ((l32 * D + (((2 * kb) ^ sw) << 3)) << 1);
        const int li = lane & 15, g = lane >> 4;
#pragma unroll
        for (int j = 0; j < D / 32; j++)
#pragma unroll
            for (int e = 0; e < 2; e++) {
                const int col = j * 32 + ((g & 1) << 4) + ((li & 3) << 2), row = 4 * (g >> 1) + (li >> 2) + 8 * e;
                ta[j][e] = lds0 + ((lds_swz_off<D>(row, col >> 3) + (col & 7)) << 1);
            }
    }
    int par = 0;
    while (have) {
        const int sk = nx_sk, pos0 = nx_pos0, key0 = nx_key0;
        t++;
        settle();
        const bool have_next = c < p.n_chunks;
        if (have_next) gload(t, par ^ 1);

        const bool need_mask = (key0 + BN > sk) || (causal && (pos0 + key0 + BN - 1 > w_lo));
        // 32 keys at a time, one block after the other: one live (S^T, dP^T) tile pair keeps the kernel at two
        // waves per SIMD, and the other wave's MFMAs cover this wave's softmax arithmetic.  A wave whose rows all
        // precede the tile's first key has nothing to add (see the forward kernel).
        if (!causal || pos0 + key0 <= w_hi) {
#pragma unroll
        for (int nb = 0; nb < BN / 32; nb++) {
            f32x16 s[RB], dp[RB];
#pragma unroll
            for (int rb = 0; rb < RB; rb++) {
                s[rb] = zero16;
                dp[rb] = ndlt[rb];
            }
            __builtin_amdgcn_s_setprio(1);   // MFMA sections run at raised priority, see the forward kernel
            lds_gemm_pair_at_rb<D, RB>(pa, nb * 32 * D * 2, TILE * 2 + nb * 32 * D * 2, qreg, doreg, s, dp);
            __builtin_amdgcn_s_setprio(0);
            // mask fix-up (tail of the chunk, diagonal tiles, rows past the end): wave-uniform branch touching S only;
            // an invisible entry gets S = -inf, so P = 0 and dS = 0
            if (need_mask) {
#pragma unroll
                for (int rb = 0; rb < RB; rb++)
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int key = key0 + nb * 32 + 8 * (r / 4) + 4 * hh + (r % 4);
                        const bool vis = key < sk && row_ok[rb] && (!causal || pos0 + key <= my_pos[rb]);
                        s[rb][r] = vis ? s[rb][r] : -INFINITY;
                    }
            }
            bf16x8 dsb[RB][2];
#pragma unroll
            for (int rb = 0; rb < RB; rb++) {
                PackedTile ds;
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    float dsv[2];
#pragma unroll
                    for (int e = 0; e < 2; e++) {
                        const int r = 2 * j + e;
                        const float pv = __builtin_amdgcn_exp2f(s[rb][r] * c2 - lse2[rb]);
                        dsv[e] = DLT_INIT ? pv * dp[rb][r] : pv * (dp[rb][r] - dlt[rb]);
                    }
                    ds.u[j] = pack2_bf16(dsv[0], dsv[1]);
                }
                dsb[rb][0] = operand_of(ds, 0);
                dsb[rb][1] = operand_of(ds, 1);
            }
            __builtin_amdgcn_s_setprio(1);
            lds_tr_gemm_at_rb<D, 2, RB>(ta, nb * 32 * D * 2, dsb, dqacc);   // every K^T operand feeds one MFMA per row block
            __builtin_amdgcn_s_setprio(0);
        }
        }
        tile_barrier();
#pragma unroll
        for (int kb = 0; kb < D / 16; kb++) pa[kb] ^= BUF_ELEMS * 2;
#pragma unroll
        for (int j = 0; j < D / 32; j++) {
            ta[j][0] ^= BUF_ELEMS * 2;
            ta[j][1] ^= BUF_ELEMS * 2;
        }
        par ^= 1;
        have = have_next;
    }

    // dQ in whole rows through the wave's LDS staging area (the tiles are no longer read: the last barrier is behind us)
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        constexpr int LPR = D / 4, ROWS_PER_IT = 64 / LPR;      // see wave_tile_rowmajor
        unsigned char *stage = smem + w * WaveStage<D>::BYTES;
        const int Sq_u = uniform32(p.Sq), wave_row0 = uniform32(row0 + w * 32 * RB + 32 * rb);
        const long long dqs1 = uniform64(p.dqs[1]);
        const long long off0 = uniform64(b * p.dqs[0] + h * p.dqs[2]) + (wave_row0 + lane / LPR) * dqs1 + 4 * (lane % LPR);
        // LTR_ROPE_DQ: q was rotated by the forward's prologue, so the gradient of the caller's un-rotated q is dQ rotated by
        // the conjugate angles of its row's position (the rotation is linear: it commutes with the accumulation over calls)
        const bool rope = uniform32(p.flags & LTR_ROPE_DQ) != 0;
        const float *const rope_tab = p.rope;
        const int rope_p0 = uniform32(p.rope_pos0), split_u = uniform32(p.q_split), qp0 = uniform32(p.q_pos0[0]), qp1 = uniform32(p.q_pos0[1]);
        auto unrotate = [&](int row, int col, f32x4 val) {
            if (!rope) return val;
            const int pos = q_position(wave_row0 + row, split_u, qp0, qp1);
            return rope_conj4(val, *(const f32x4 *)(rope_tab + (long long)(pos - rope_p0) * D + col));
        };
        if (uniform32(p.flags & LTR_DQ_BF16)) {   // this call saw every key of these rows: store the result, no accumulator
            __bf16 *dqp = (__bf16 *)p.dq + off0;
            wave_tile_rowmajor<D>(stage, lane, dqacc[rb], p.scale, [&](int row, int col, f32x4 val) {
                if (wave_row0 + row < Sq_u) {
                    val = unrotate(row, col, val);
                    bf16x4 y;
#pragma unroll
                    for (int e = 0; e < 4; e++) y[e] = (__bf16)val[e];
                    *(bf16x4 *)dqp = y;
                }
                dqp += ROWS_PER_IT * dqs1;
            });
        } else {
            float *dqp = (float *)p.dq + off0;
            constexpr int NIT = 32 / ROWS_PER_IT;
            f32x4 old[NIT];   // all reads of the accumulator first, then the adds and the writes
#pragma unroll
            for (int it = 0; it < NIT; it++) {
                old[it] = f32x4{0.f, 0.f, 0.f, 0.f};
                if (wave_row0 + it * ROWS_PER_IT + lane / LPR < Sq_u) old[it] = *(const f32x4 *)(dqp + it * ROWS_PER_IT * dqs1);
            }
            int it = 0;
            wave_tile_rowmajor<D>(stage, lane, dqacc[rb], p.scale, [&](int row, int col, f32x4 val) {
                if (wave_row0 + row < Sq_u) {
                    val = unrotate(row, col, val);
#pragma unroll
                    for (int e = 0; e < 4; e++) val[e] += old[it][e];
                    *(f32x4 *)dqp = val;
                }
                dqp += ROWS_PER_IT * dqs1;
                it++;
            });
        }
    }
    }   // part
}

// ------------------------------------------------------------------------------ backward, fp32
// The fp32 path (1e-4 parity cases, not a performance path): scalar FMAs like fwd_f32_kernel, no atomics.
//   bwd_dq_f32_kernel    one query row per lane (q, dO, dQ in registers), K/V tiles of 32 keys broadcast from LDS
//   bwd_dkdv_f32_kernel  one key per lane, Q/dO tiles of 32 rows (+ LSE, DELTA) broadcast from LDS; two passes so that
//                        the per-lane state fits the register file: DV = false keeps K, V, dK; DV = true keeps K, dV
template <int D>
__global__ __launch_bounds__(64) void bwd_dq_f32_kernel(const BwdParams p) {
    constexpr int BN = 32;
    __shared__ __attribute__((aligned(16))) float Ks[BN * D];
    __shared__ __attribute__((aligned(16))) float Vs[BN * D];
    const int tid = threadIdx.x;
    const bool causal = p.flags & LTR_CAUSAL;
    const int n_qt = (p.Sq + 63) / 64;
    const int qt = n_qt - 1 - (int)(blockIdx.x % n_qt), bh = blockIdx.x / n_qt;
    const int b = bh / p.Hq, h = bh % p.Hq, hkv = h / p.n_rep;
    const int row0 = qt * 64, my_row = row0 + tid;
    const bool row_ok = my_row < p.Sq;
    const int my_pos = q_position(my_row, p.q_split, p.q_pos0[0], p.q_pos0[1]);
    int blk_lo, blk_hi;
    q_pos_range(row0, min(row0 + 64, p.Sq) - 1, p.q_split, p.q_pos0[0], p.q_pos0[1], blk_lo, blk_hi);

    // the accumulator covers 64 (D = 128: 32) elements of the head dimension at a time, one pass over the keys each, so that the
    // per-lane state stays inside the register file
    constexpr int DP = D == 128 ? 32 : 64;
    float q[D], dO[D], dq[DP];
    float lse = INFINITY, dlt = 0.f;   // +inf: P = exp(s - inf) = 0 for rows past the end and rows that saw no key
    {
        const int rs = min(my_row, p.Sq - 1);
        const float *qp = (const float *)p.q + b * p.qs[0] + (long long)rs * p.qs[1] + h * p.qs[2];
        const float *dop = (const float *)p.d_o + b * p.dos[0] + (long long)rs * p.dos[1] + h * p.dos[2];
#pragma unroll
        for (int d = 0; d < D; d++) {
            q[d] = qp[d];
            dO[d] = dop[d];
        }
        if (row_ok) {
            const float l = p.lse[((long long)b * p.Hq + h) * p.Sq + my_row];
            lse = l == -INFINITY ? INFINITY : l;
            dlt = p.delta[((long long)b * p.Hq + h) * p.Sq + my_row];
        }
    }
    for (int part = 0; part < D / DP; part++) {
#pragma unroll
    for (int d = 0; d < DP; d++) dq[d] = 0.f;
    for (int c = 0; c < p.n_chunks; c++) {
        const int sk = p.chunk[c].sk, pos0 = p.chunk[c].pos0;
        const int nvis = causal ? max(0, min(sk, blk_hi - pos0 + 1)) : sk;
        const float *kp = (const float *)p.chunk[c].k + b * p.ks[0] + hkv * p.ks[2];
        const float *vp = (const float *)p.chunk[c].v + b * p.vs[0] + hkv * p.vs[2];
        for (int key0 = 0; key0 < nvis; key0 += BN) {
            __syncthreads();
            for (int i = tid; i < BN * D / 4; i += 64) {
                const int key = key0 + i / (D / 4), dc = i % (D / 4);
                f32x4 kv = {0.f, 0.f, 0.f, 0.f}, vv = {0.f, 0.f, 0.f, 0.f};
                if (key < sk) {
                    kv = *(const f32x4 *)(kp + (long long)key * p.ks[1] + dc * 4);
                    vv = *(const f32x4 *)(vp + (long long)key * p.vs[1] + dc * 4);
                }
                *(f32x4 *)(Ks + i * 4) = kv;
                *(f32x4 *)(Vs + i * 4) = vv;
            }
            __syncthreads();
#pragma unroll 1
            for (int j = 0; j < BN; j++) {
                float s = 0.f, dp = 0.f;
#pragma unroll
                for (int d4 = 0; d4 < D / 4; d4++) {
                    const f32x4 kq = *(const f32x4 *)(Ks + j * D + 4 * d4), vq = *(const f32x4 *)(Vs + j * D + 4 * d4);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        s = fmaf(q[4 * d4 + e], kq[e], s);
                        dp = fmaf(dO[4 * d4 + e], vq[e], dp);
                    }
                    if ((d4 & 7) == 7) asm volatile("" ::: "memory");   // bounds the LDS reads in flight (registers)
                }
                const int key = key0 + j;
                const bool vis = key < sk && (!causal || pos0 + key <= my_pos);
                const float pj = vis ? expf(s * p.scale - lse) : 0.f;
                const float ds = pj * (dp - dlt);
#pragma unroll
                for (int d = 0; d < DP; d++) dq[d] = fmaf(ds, Ks[j * D + part * DP + d], dq[d]);
            }
        }
    }
    if (row_ok) {
        float *dqp = (float *)p.dq + b * p.dqs[0] + (long long)my_row * p.dqs[1] + h * p.dqs[2] + part * DP;
#pragma unroll
        for (int d = 0; d < DP; d++) dqp[d] += dq[d] * p.scale;
    }
    }
}

template <int D, bool DV>
__global__ __launch_bounds__(64) void bwd_dkdv_f32_kernel(const BwdParams p) {
    constexpr int BM = 32;
    __shared__ __attribute__((aligned(16))) float Qs[BM * D];
    __shared__ __attribute__((aligned(16))) float dOs[BM * D];
    __shared__ float lse_s[BM], dlt_s[BM];
    const int tid = threadIdx.x;
    const bool causal = p.flags & LTR_CAUSAL;
    // block -> (batch, kv head, chunk, 64-key tile)
    const int P = p.B * p.Hkv;
    const int pair = blockIdx.x % P;
    int kt = blockIdx.x / P;
    const int b = pair / p.Hkv, hkv = pair % p.Hkv;
    int c = 0;
    for (; c < p.n_chunks; c++) {
        const int n = (p.chunk[c].sk + 63) / 64;
        if (kt < n) break;
        kt -= n;
    }
    if (c >= p.n_chunks) return;
    const int sk = p.chunk[c].sk, pos0 = p.chunk[c].pos0;
    const int my_key = kt * 64 + tid;
    const bool key_ok = my_key < sk;
    const int my_kpos = pos0 + my_key, tile_kpos_lo = pos0 + kt * 64;

    constexpr int DP = D == 128 ? 32 : 64;   // see bwd_dq_f32_kernel
    float k[D], v[DV ? 1 : D], acc[DP];
    {
        const int ks_ = min(my_key, sk - 1);
        const float *kp = (const float *)p.chunk[c].k + b * p.ks[0] + (long long)ks_ * p.ks[1] + hkv * p.ks[2];
        const float *vp = (const float *)p.chunk[c].v + b * p.vs[0] + (long long)ks_ * p.vs[1] + hkv * p.vs[2];
#pragma unroll
        for (int d = 0; d < D; d++) {
            k[d] = kp[d];
            if (!DV) v[d] = vp[d];
        }
    }
    for (int part = 0; part < D / DP; part++) {
#pragma unroll
    for (int d = 0; d < DP; d++) acc[d] = 0.f;
    for (int rep = 0; rep < p.n_rep; rep++) {
        const int h = hkv * p.n_rep + rep;
        const float *qp = (const float *)p.q + b * p.qs[0] + h * p.qs[2];
        const float *dop = (const float *)p.d_o + b * p.dos[0] + h * p.dos[2];
        const long long so = ((long long)b * p.Hq + h) * p.Sq;
        for (int row0 = 0; row0 < p.Sq; row0 += BM) {
            if (causal) {   // no row of the tile sees any key of the block
                int lo, hi;
                q_pos_range(row0, min(row0 + BM, p.Sq) - 1, p.q_split, p.q_pos0[0], p.q_pos0[1], lo, hi);
                if (hi < tile_kpos_lo) continue;
            }
            __syncthreads();
            for (int i = tid; i < BM * D / 4; i += 64) {
                const int row = row0 + i / (D / 4), dc = i % (D / 4);
                f32x4 qv = {0.f, 0.f, 0.f, 0.f}, dv = {0.f, 0.f, 0.f, 0.f};
                if (row < p.Sq) {
                    qv = *(const f32x4 *)(qp + (long long)row * p.qs[1] + dc * 4);
                    dv = *(const f32x4 *)(dop + (long long)row * p.dos[1] + dc * 4);
                }
                *(f32x4 *)(Qs + i * 4) = qv;
                *(f32x4 *)(dOs + i * 4) = dv;
            }
            if (tid < BM) {
                const int row = row0 + tid;
                const float l = row < p.Sq ? p.lse[so + row] : INFINITY;
                lse_s[tid] = l == -INFINITY ? INFINITY : l;     // +inf: P = 0
                dlt_s[tid] = row < p.Sq ? p.delta[so + row] : 0.f;
            }
            __syncthreads();
#pragma unroll 1
            for (int i = 0; i < BM; i++) {
                float s = 0.f, dp = 0.f;
#pragma unroll
                for (int d4 = 0; d4 < D / 4; d4++) {
                    const f32x4 qq = *(const f32x4 *)(Qs + i * D + 4 * d4);
                    f32x4 oq = {0.f, 0.f, 0.f, 0.f};
                    if (!DV) oq = *(const f32x4 *)(dOs + i * D + 4 * d4);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        s = fmaf(k[4 * d4 + e], qq[e], s);
                        if (!DV) dp = fmaf(v[4 * d4 + e], oq[e], dp);
                    }
                    if ((d4 & 7) == 7) asm volatile("" ::: "memory");   // bounds the LDS reads in flight (registers)
                }
                const int qpos = q_position(row0 + i, p.q_split, p.q_pos0[0], p.q_pos0[1]);
                const bool vis = key_ok && (!causal || my_kpos <= qpos);
                const float pi = vis ? expf(s * p.scale - lse_s[i]) : 0.f;
                if (DV) {
#pragma unroll
                    for (int d = 0; d < DP; d++) acc[d] = fmaf(pi, dOs[i * D + part * DP + d], acc[d]);
                } else {
                    const float ds = pi * (dp - dlt_s[i]);
#pragma unroll
                    for (int d = 0; d < DP; d++) acc[d] = fmaf(ds, Qs[i * D + part * DP + d], acc[d]);
                }
            }
        }
    }
    if (key_ok) {
        float *gp = (DV ? p.chunk[c].dv + b * p.dvs[0] + (long long)my_key * p.dvs[1] + hkv * p.dvs[2]
                        : p.chunk[c].dk + b * p.dks[0] + (long long)my_key * p.dks[1] + hkv * p.dks[2]) + part * DP;
        const float mul = DV ? 1.f : p.scale;
#pragma unroll
        for (int d = 0; d < DP; d++) gp[d] += acc[d] * mul;
    }
    }
}

// ------------------------------------------------------------------------------ backward, fp32 on the matrix pipe
// The recompute backward of the fp32 path on v_mfma_f32_32x32x2_f32, in the shapes of fwd_f32_mfma_kernel (same LDS-direct
// swizzled fp32 tiles, same choice of contraction order so that no operand moves), no atomics:
//   bwd_dq_f32_mfma_kernel<D, KS>   4 waves, a wave owns 32 query rows (lane = row; Q, dO operands in registers) and one of
//                        KS key shares: S^T = K Q^T and dP^T = V dO^T (accumulators start at -DELTA), dS^T = P (dP - DELTA)
//                        in registers, dQ^T += K^T dS^T with the accumulator register as the step's operand; the KS partial
//                        dQ of a row group are summed through LDS; dQ is added to the fp32 accumulator in whole rows.
//   bwd_dkdv_f32_mfma_kernel<D>     4 waves, a wave owns 32 keys (lane = key; K, V operands and the dK^T, dV^T accumulators
//                        in registers: one wave per SIMD), the block loops over the group's query heads and over 32-row
//                        Q / dO tiles in double-buffered LDS: S = Q K^T, dP = dO V^T (accumulators start at -DELTA of
//                        their rows), P and dS in registers, dV^T += dO^T P, dK^T += Q^T dS.
template <int D, int KS>
__global__ __launch_bounds__(256) void bwd_dq_f32_mfma_kernel(const BwdParams p) {
    using L = F32Mfma<D, KS>;
    constexpr int NW = L::NW, RG = L::RG, BM = L::BM, BN = L::BN, TILE = L::TILE;
    constexpr int CPR = D / 4, RPI = 64 / CPR, NI = BN / (RPI * NW);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, hh = lane >> 5;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rg = w / KS, ks = w % KS;
    const bool causal = p.flags & LTR_CAUSAL;
    const int n_qt = (p.Sq + BM - 1) / BM;
    const int idx = blockIdx.x;
    const int qt = n_qt - 1 - idx / (p.B * p.Hq);
    const int bh = idx % (p.B * p.Hq);
    const int b = bh / p.Hq, h = bh % p.Hq, hkv = h / p.n_rep;
    const int row0 = qt * BM, my_row = row0 + rg * 32 + l32;
    const bool row_ok = my_row < p.Sq;
    const int my_pos = q_position(my_row, p.q_split, p.q_pos0[0], p.q_pos0[1]);
    int blk_lo, blk_hi, w_lo, w_hi;
    q_pos_range(row0, min(row0 + BM, p.Sq) - 1, p.q_split, p.q_pos0[0], p.q_pos0[1], blk_lo, blk_hi);
    {
        const int wr0 = row0 + rg * 32, wr1 = min(wr0 + 32, p.Sq) - 1;
        if (wr1 >= wr0) q_pos_range(wr0, wr1, p.q_split, p.q_pos0[0], p.q_pos0[1], w_lo, w_hi);
        else { w_lo = 0x7fffffff; w_hi = -0x7fffffff; }
    }
    // operands of the lane's row: qreg[4g + j] = Q[row][8g + 4h + j], doreg likewise
    float qreg[D / 2], doreg[D / 2];
    float lse2 = INFINITY, dlt = 0.f;   // +inf: P = exp2(s - inf) = 0 for rows past the end and rows that saw no key
    {
        const int rs = min(my_row, p.Sq - 1);
        const float *qp = (const float *)p.q + b * p.qs[0] + (long long)rs * p.qs[1] + h * p.qs[2];
        const float *dop = (const float *)p.d_o + b * p.dos[0] + (long long)rs * p.dos[1] + h * p.dos[2];
#pragma unroll
        for (int g = 0; g < D / 8; g++) {
            const f32x4 x = *(const f32x4 *)(qp + 8 * g + 4 * hh), y = *(const f32x4 *)(dop + 8 * g + 4 * hh);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                qreg[4 * g + j] = x[j];
                doreg[4 * g + j] = y[j];
            }
        }
        if (row_ok) {
            const float lse_row = p.lse[((long long)b * p.Hq + h) * p.Sq + my_row];
            lse2 = lse_row == -INFINITY ? INFINITY : lse_row * LTR_LOG2E;
            dlt = p.delta[((long long)b * p.Hq + h) * p.Sq + my_row];
        }
    }
    f32x16 dqacc[D / 32], ndlt;
#pragma unroll
    for (int r = 0; r < 16; r++) ndlt[r] = -dlt;
#pragma unroll
    for (int i = 0; i < D / 32; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) dqacc[i][r] = 0.f;
    const float c2 = p.scale * LTR_LOG2E;

    int c = -1, t = 0, nt = 0;
    int ld_sk = 0, ld_pos0 = 0;
    const float *ld_kb = nullptr, *ld_vb = nullptr;
    auto settle = [&]() {
        while (c < p.n_chunks && t >= nt) {
            c++;
            t = 0;
            if (c < p.n_chunks) {
                ld_sk = p.chunk[c].sk;
                ld_pos0 = p.chunk[c].pos0;
                ld_kb = (const float *)p.chunk[c].k + b * p.ks[0] + hkv * p.ks[2];
                ld_vb = (const float *)p.chunk[c].v + b * p.vs[0] + hkv * p.vs[2];
                const int nvis = causal ? max(0, min(ld_sk, blk_hi - ld_pos0 + 1)) : ld_sk;
                nt = (nvis + BN - 1) / BN;
            }
        }
    };
    settle();
    const int st_row = lane / CPR, st_pc = lane % CPR;
    int nx_sk = 0, nx_pos0 = 0, nx_key0 = 0;
    auto gload = [&](int ti, int buf) {
        nx_sk = ld_sk;
        nx_pos0 = ld_pos0;
        nx_key0 = ti * BN;
        const unsigned Kd = lds_address(smem) + buf * L::BUF_BYTES, Vd = Kd + TILE * 4;
#pragma unroll
        for (int i = 0; i < NI; i++) {
            const int row = RPI * (NI * w + i) + st_row;
            const int key = min(ti * BN + row, ld_sk - 1);
            const int chunk = st_pc ^ f32_swz(row);
            global_to_lds_b128(ld_kb + ((long long)key * p.ks[1] + chunk * 4), Kd + RPI * (NI * w + i) * D * 4);
            global_to_lds_b128(ld_vb + ((long long)key * p.vs[1] + chunk * 4), Vd + RPI * (NI * w + i) * D * 4);
        }
    };
    bool have = c < p.n_chunks;
    if (!have) return;              // no visible key: nothing to add to the accumulator (block-uniform)
    gload(t, 0);
    tile_barrier();
    int par = 0;
    while (have) {
        const int sk = nx_sk, pos0 = nx_pos0, key0 = nx_key0 + 32 * ks;
        const float *Ks = (const float *)(smem + par * L::BUF_BYTES) + 32 * ks * D, *Vs = Ks + TILE;
        t++;
        settle();
        const bool have_next = c < p.n_chunks;
        if (have_next) gload(t, par ^ 1);
        if (key0 < sk && (!causal || pos0 + key0 <= w_hi)) {
            f32x16 s, dp = ndlt;
#pragma unroll
            for (int r = 0; r < 16; r++) s[r] = 0.f;
            const float *krow = Ks + l32 * D, *vrow_ = Vs + l32 * D;
            const int ksw = f32_swz(l32);
#pragma unroll
            for (int g = 0; g < D / 8; g++) {
                const f32x4 kx = *(const f32x4 *)(krow + (((2 * g + hh) ^ ksw) << 2));
                const f32x4 vx = *(const f32x4 *)(vrow_ + (((2 * g + hh) ^ ksw) << 2));
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    s = __builtin_amdgcn_mfma_f32_32x32x2f32(kx[j], qreg[4 * g + j], s, 0, 0, 0);
                    dp = __builtin_amdgcn_mfma_f32_32x32x2f32(vx[j], doreg[4 * g + j], dp, 0, 0, 0);
                }
            }
            const bool need_mask = (key0 + 32 > sk) || (causal && (pos0 + key0 + 31 > w_lo));
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float pv = __builtin_amdgcn_exp2f(s[r] * c2 - lse2);
                if (need_mask) {
                    const int key = key0 + 8 * (r / 4) + 4 * hh + (r % 4);
                    const bool vis = key < sk && row_ok && (!causal || pos0 + key <= my_pos);
                    pv = vis ? pv : 0.f;
                }
                s[r] = pv * dp[r];          // dS^T, key 8 (r / 4) + 4h + r % 4 of the sub-tile
            }
            // dQ^T += K^T dS^T: step r contracts the key of accumulator register r; lane (d = 32 db + l32, h) reads K[key][d]
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int krow_i = 8 * (r / 4) + 4 * hh + (r % 4);
                const float *kr = Ks + krow_i * D + (l32 & 3);
                const int sw = f32_swz(krow_i);
#pragma unroll
                for (int db = 0; db < D / 32; db++) {
                    const float kx = kr[((8 * db + (l32 >> 2)) ^ sw) << 2];
                    dqacc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(kx, s[r], dqacc[db], 0, 0, 0);
                }
            }
        }
        tile_barrier();
        par ^= 1;
        have = have_next;
    }
    // sum of the KS partial dQ of a row group
    if constexpr (KS > 1) {
        float *part = (float *)(smem + L::PART_OFF);
        if (ks > 0) {
            float *mine = part + (size_t)(rg * (KS - 1) + ks - 1) * (L::PART_BYTES / 4);
#pragma unroll
            for (int i = 0; i < D / 32; i++)
#pragma unroll
                for (int r4 = 0; r4 < 4; r4++) {
                    f32x4 x;
#pragma unroll
                    for (int e = 0; e < 4; e++) x[e] = dqacc[i][4 * r4 + e];
                    *(f32x4 *)(mine + ((i * 4 + r4) * 64 + lane) * 4) = x;
                }
        }
        __syncthreads();
        if (ks > 0) return;
        for (int k2 = 1; k2 < KS; k2++) {
            const float *other = part + (size_t)(rg * (KS - 1) + k2 - 1) * (L::PART_BYTES / 4);
#pragma unroll
            for (int i = 0; i < D / 32; i++)
#pragma unroll
                for (int r4 = 0; r4 < 4; r4++) {
                    const f32x4 x = *(const f32x4 *)(other + ((i * 4 + r4) * 64 + lane) * 4);
#pragma unroll
                    for (int e = 0; e < 4; e++) dqacc[i][4 * r4 + e] += x[e];
                }
        }
    }
    unsigned char *stage = smem + L::STAGE_OFF + rg * WaveStage<D>::BYTES;
    constexpr int LPR = D / 4, ROWS_PER_IT = 64 / LPR;
    const int wave_row0 = row0 + rg * 32, Sq = p.Sq;
    const long long dqs1 = p.dqs[1];
    float *dqp = (float *)p.dq + b * p.dqs[0] + h * p.dqs[2] + (long long)(wave_row0 + lane / LPR) * dqs1 + 4 * (lane % LPR);
    wave_tile_rowmajor<D>(stage, lane, dqacc, p.scale, [&](int row, int, f32x4 val) {
        if (wave_row0 + row < Sq) {
            const f32x4 old = *(const f32x4 *)dqp;
#pragma unroll
            for (int e = 0; e < 4; e++) val[e] += old[e];
            *(f32x4 *)dqp = val;
        }
        dqp += ROWS_PER_IT * dqs1;
    });
}

template <int D>
struct F32DkdvLds {
    static constexpr int TILE = 32 * D;                          // floats per Q (or dO) tile of 32 rows
    static constexpr int BUF_BYTES = 2 * TILE * 4 + 3 * 32 * 4;  // Q, dO, LSE * log2(e), -DELTA, row positions
    static constexpr int STAGE_BYTES = 4 * WaveStage<D>::BYTES;
    static constexpr int LDS = 2 * BUF_BYTES > STAGE_BYTES ? 2 * BUF_BYTES : STAGE_BYTES;
};

template <int D>
__global__ __launch_bounds__(256) void bwd_dkdv_f32_mfma_kernel(const BwdParams p) {
    using L = F32DkdvLds<D>;
    constexpr int BN = 128, BM = 32, TILE = L::TILE;
    constexpr int CPR = D / 4, RPI = 64 / CPR, NI = BM / (RPI * 4);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, hh = lane >> 5;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool causal = p.flags & LTR_CAUSAL;
    // block -> (batch, kv head, chunk, 128-key tile)
    const int P = p.B * p.Hkv;
    const int pair = blockIdx.x % P;
    int c = 0, kt = blockIdx.x / P;
    for (; c < p.n_chunks; c++) {
        const int n = (p.chunk[c].sk + BN - 1) / BN;
        if (kt < n) break;
        kt -= n;
    }
    if (c >= p.n_chunks) return;
    const int b = pair / p.Hkv, hkv = pair % p.Hkv;
    const int sk = p.chunk[c].sk, pos0 = p.chunk[c].pos0;
    const int key0 = kt * BN, my_key = key0 + 32 * w + l32;
    const bool key_ok = my_key < sk;
    const int kpos = key_ok ? pos0 + my_key : BWD_KPOS_NONE;
    const int blk_kpos_lo = pos0 + key0, w_kpos_lo = pos0 + key0 + 32 * w;
    if (causal) {   // no query of this launch sees the block
        int q_lo, q_hi;
        q_pos_range(0, (int)p.Sq - 1, p.q_split, p.q_pos0[0], p.q_pos0[1], q_lo, q_hi);
        if (q_hi < blk_kpos_lo) return;
    }
    // operands of the lane's key: kreg[4g + j] = K[key][8g + 4h + j], vreg likewise
    float kreg[D / 2], vreg[D / 2];
    {
        const int ksafe = min(my_key, sk - 1);
        const float *kp = (const float *)p.chunk[c].k + b * p.ks[0] + (long long)ksafe * p.ks[1] + hkv * p.ks[2];
        const float *vp = (const float *)p.chunk[c].v + b * p.vs[0] + (long long)ksafe * p.vs[1] + hkv * p.vs[2];
#pragma unroll
        for (int g = 0; g < D / 8; g++) {
            f32x4 x = *(const f32x4 *)(kp + 8 * g + 4 * hh), y = *(const f32x4 *)(vp + 8 * g + 4 * hh);
            if (!key_ok) x = y = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                kreg[4 * g + j] = x[j];
                vreg[4 * g + j] = y[j];
            }
        }
    }
    f32x16 dkacc[D / 32], dvacc[D / 32];
#pragma unroll
    for (int i = 0; i < D / 32; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) dkacc[i][r] = dvacc[i][r] = 0.f;
    const float c2 = p.scale * LTR_LOG2E;

    // walk over (query head of the group, 32-row q tile); tiles none of whose rows sees a key of the block are skipped
    const int n_qt = (p.Sq + BM - 1) / BM, total = p.n_rep * n_qt;
    auto visible = [&](int it) {
        if (!causal) return true;
        const int r0 = (it % n_qt) * BM;
        int lo, hi;
        q_pos_range(r0, min(r0 + BM, p.Sq) - 1, p.q_split, p.q_pos0[0], p.q_pos0[1], lo, hi);
        return hi >= blk_kpos_lo;
    };
    auto next_visible = [&](int it) {
        while (it < total && !visible(it)) it++;
        return it;
    };
    const int st_row = lane / CPR, st_pc = lane % CPR;
    auto gload = [&](int it, int buf) {
        const int rep = it / n_qt, r0 = (it % n_qt) * BM, h = hkv * p.n_rep + rep;
        const float *qp = (const float *)p.q + b * p.qs[0] + h * p.qs[2];
        const float *dop = (const float *)p.d_o + b * p.dos[0] + h * p.dos[2];
        const unsigned Qd = lds_address(smem) + buf * L::BUF_BYTES, dOd = Qd + TILE * 4;
#pragma unroll
        for (int i = 0; i < NI; i++) {
            const int row = RPI * (NI * w + i) + st_row;
            const int grow = min(r0 + row, p.Sq - 1);
            const int chunk = st_pc ^ f32_swz(row);
            global_to_lds_b128(qp + ((long long)grow * p.qs[1] + chunk * 4), Qd + RPI * (NI * w + i) * D * 4);
            global_to_lds_b128(dop + ((long long)grow * p.dos[1] + chunk * 4), dOd + RPI * (NI * w + i) * D * 4);
        }
        // per-row scalars of the tile: LSE * log2(e) (+inf for rows past the end or without a visible key), -DELTA, position
        float *st = (float *)(smem + buf * L::BUF_BYTES) + 2 * TILE;
        if (tid < 96) {
            const int r = tid & 31, row = r0 + r;
            const bool ok = row < p.Sq;
            const long long so = ((long long)b * p.Hq + h) * p.Sq + min(row, p.Sq - 1);
            if (tid < 32) {
                const float l = p.lse[so];
                st[r] = (!ok || l == -INFINITY) ? INFINITY : l * LTR_LOG2E;
            } else if (tid < 64) {
                st[32 + r] = ok ? -p.delta[so] : 0.f;
            } else {
                ((int *)st)[64 + r] = !ok ? BWD_QPOS_NONE : causal ? q_position(row, p.q_split, p.q_pos0[0], p.q_pos0[1]) : BWD_QPOS_ALL;
            }
        }
    };
    int it = next_visible(0);
    if (it < total) gload(it, 0);
    tile_barrier();
    int par = 0;
    while (it < total) {
        const int nxt = next_visible(it + 1);
        if (nxt < total) gload(nxt, par ^ 1);
        const float *Qs = (const float *)(smem + par * L::BUF_BYTES), *dOs = Qs + TILE;
        const float *st = dOs + TILE;
        // a wave whose 32 keys no row of the tile sees has nothing to add
        int lo, hi;
        {
            const int r0 = (it % n_qt) * BM;
            q_pos_range(r0, min(r0 + BM, p.Sq) - 1, p.q_split, p.q_pos0[0], p.q_pos0[1], lo, hi);
        }
        if (!causal || hi >= w_kpos_lo) {
            f32x16 s, dp;
            float lse2[16];
            int qpos[16];
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const f32x4 a = *(const f32x4 *)(st + 8 * g + 4 * hh), d4 = *(const f32x4 *)(st + 32 + 8 * g + 4 * hh);
                const i32x4 q4 = *(const i32x4 *)((const int *)st + 64 + 8 * g + 4 * hh);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    lse2[4 * g + e] = a[e];
                    dp[4 * g + e] = d4[e];      // the dP accumulator starts at -DELTA of its row
                    qpos[4 * g + e] = q4[e];
                    s[4 * g + e] = 0.f;
                }
            }
            const float *qrow = Qs + l32 * D, *dorow = dOs + l32 * D;
            const int rsw = f32_swz(l32);
#pragma unroll
            for (int g = 0; g < D / 8; g++) {
                const f32x4 qx = *(const f32x4 *)(qrow + (((2 * g + hh) ^ rsw) << 2));
                const f32x4 dx = *(const f32x4 *)(dorow + (((2 * g + hh) ^ rsw) << 2));
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    s = __builtin_amdgcn_mfma_f32_32x32x2f32(qx[j], kreg[4 * g + j], s, 0, 0, 0);
                    dp = __builtin_amdgcn_mfma_f32_32x32x2f32(dx[j], vreg[4 * g + j], dp, 0, 0, 0);
                }
            }
            // register r <-> tile row 8 (r / 4) + 4h + r % 4, lane <-> key: P and dS of the (row, key) pair
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float pv = __builtin_amdgcn_exp2f(s[r] * c2 - lse2[r]);
                pv = kpos <= qpos[r] ? pv : 0.f;
                s[r] = pv;
                dp[r] = pv * dp[r];
            }
            // dV^T += dO^T P and dK^T += Q^T dS: step r contracts the row of accumulator register r; lane (d = 32 db + l32, h)
            // reads dO[row][d] / Q[row][d]
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int trow = 8 * (r / 4) + 4 * hh + (r % 4);
                const int sw = f32_swz(trow);
                const float *dor = dOs + trow * D + (l32 & 3), *qr = Qs + trow * D + (l32 & 3);
#pragma unroll
                for (int db = 0; db < D / 32; db++) {
                    const int off = ((8 * db + (l32 >> 2)) ^ sw) << 2;
                    dvacc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(dor[off], s[r], dvacc[db], 0, 0, 0);
                    dkacc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(qr[off], dp[r], dkacc[db], 0, 0, 0);
                }
            }
        }
        tile_barrier();
        par ^= 1;
        it = nxt;
    }
    // dK^T / dV^T of the wave's 32 keys: added to the fp32 accumulators in whole rows through the wave's staging area
    unsigned char *stage = smem + w * WaveStage<D>::BYTES;
    constexpr int LPR = D / 4, ROWS_PER_IT = 64 / LPR;
    const int key_base = key0 + 32 * w;
    auto add_rows = [&](const f32x16 (&acc)[D / 32], float mul, float *base, long long stride) {
        float *gp = base + (long long)(key_base + lane / LPR) * stride + 4 * (lane % LPR);
        wave_tile_rowmajor<D>(stage, lane, acc, mul, [&](int row, int, f32x4 val) {
            if (key_base + row < sk) {
                const f32x4 old = *(const f32x4 *)gp;
#pragma unroll
                for (int e = 0; e < 4; e++) val[e] += old[e];
                *(f32x4 *)gp = val;
            }
            gp += ROWS_PER_IT * stride;
        });
    };
    add_rows(dkacc, p.scale, p.chunk[c].dk + b * p.dks[0] + hkv * p.dks[2], p.dks[1]);
    add_rows(dvacc, 1.f, p.chunk[c].dv + b * p.dvs[0] + hkv * p.dvs[2], p.dvs[1]);
}

// ------------------------------------------------------------------------------ host side
bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

// Per-device facts, found out on the first call on each device and read-only afterwards.  The fields are atomics: two host
// threads that make their first call at the same time both do the (idempotent) work and store the same answer.  A failed
// query or opt-in is not remembered: the next call tries again.
constexpr int LTR_MAX_DEVICES = 64;
struct DeviceState {
    std::atomic<int> arch{0};          // 0 unknown, 1 gfx950, -1 something else
    std::atomic<int> large_lds{0};     // 1: the kernels of this device may use more than 64 KB of dynamic LDS
    std::atomic<int> cus{0};           // compute units (0: not asked yet)
    std::atomic<float *> scratch{nullptr};   // device address of this device's copy of `scratch`
};
DeviceState g_dev[LTR_MAX_DEVICES];

int current_device(int *dev) {
    if (hipGetDevice(dev) != hipSuccess || *dev < 0 || *dev >= LTR_MAX_DEVICES) return LTR_EDEVICE;
    return LTR_OK;
}

int check_device() {   // gfx950 only
    int dev = 0;
    if (current_device(&dev)) return LTR_EDEVICE;
    int arch = g_dev[dev].arch.load(std::memory_order_acquire);
    if (arch == 0) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return LTR_EDEVICE;
        const char *a = prop.gcnArchName;
        arch = (a[0] == 'g' && a[1] == 'f' && a[2] == 'x' && a[3] == '9' && a[4] == '5' && a[5] == '0') ? 1 : -1;
        g_dev[dev].arch.store(arch, std::memory_order_release);
    }
    return arch == 1 ? LTR_OK : LTR_EDEVICE;
}

// kernels that need more than 64 KB of dynamic LDS must opt in once per device
template <int D, int RB = 1>
constexpr int fwd_lds_bytes() {   // the K / V tile buffers, reused by the epilogue's staging areas (one per wave)
    return 2 * 2 * FwdTile<D, RB>::BN * D * 2 > 8 * WaveStage<D>::BYTES ? 2 * 2 * FwdTile<D, RB>::BN * D * 2 : 8 * WaveStage<D>::BYTES;
}
template <int D>
constexpr int dq_lds_bytes() { return fwd_lds_bytes<D>(); }   // same tile buffers and staging areas as the forward

int enable_large_lds() {
    int dev = 0;
    if (current_device(&dev)) return LTR_EDEVICE;
    if (g_dev[dev].large_lds.load(std::memory_order_acquire) == 1) return LTR_OK;
    bool ok = hipFuncSetAttribute((const void *)bwd_dkdv_kernel<128, 1>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  BwdLds<128, 1>::TOTAL) == hipSuccess &&
              hipFuncSetAttribute((const void *)bwd_dkdv_kernel<64, 1>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  BwdLds<64, 1>::TOTAL) == hipSuccess &&
              hipFuncSetAttribute((const void *)bwd_dkdv_kernel<64, 2>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  BwdLds<64, 2>::TOTAL) == hipSuccess &&
              hipFuncSetAttribute((const void *)fwd_bf16_kernel<128, 1>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  fwd_lds_bytes<128>()) == hipSuccess &&
              hipFuncSetAttribute((const void *)fwd_bf16_kernel<64, 1>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  fwd_lds_bytes<64>()) == hipSuccess &&
              hipFuncSetAttribute((const void *)fwd_bf16_kernel<64, 2>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  fwd_lds_bytes<64, 2>()) == hipSuccess &&
              hipFuncSetAttribute((const void *)bwd_dq_kernel<128, 1>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  dq_lds_bytes<128>()) == hipSuccess &&
              hipFuncSetAttribute((const void *)bwd_dq_kernel<64, 1>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  dq_lds_bytes<64>()) == hipSuccess &&
              hipFuncSetAttribute((const void *)bwd_dq_kernel<64, 2>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  dq_lds_bytes<64>()) == hipSuccess &&
              hipFuncSetAttribute((const void *)fwd_f32_mfma_kernel<128, 1>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  F32Mfma<128, 1>::LDS) == hipSuccess &&
              hipFuncSetAttribute((const void *)fwd_f32_mfma_kernel<128, 2>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  F32Mfma<128, 2>::LDS) == hipSuccess &&
              hipFuncSetAttribute((const void *)fwd_f32_mfma_kernel<64, 1>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  F32Mfma<64, 1>::LDS) == hipSuccess &&
              hipFuncSetAttribute((const void *)fwd_f32_mfma_kernel<64, 2>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  F32Mfma<64, 2>::LDS) == hipSuccess &&
              hipFuncSetAttribute((const void *)fwd_f32_mfma_kernel<64, 4>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  F32Mfma<64, 4>::LDS) == hipSuccess &&
              hipFuncSetAttribute((const void *)bwd_dq_f32_mfma_kernel<128, 1>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  F32Mfma<128, 1>::LDS) == hipSuccess &&
              hipFuncSetAttribute((const void *)bwd_dq_f32_mfma_kernel<128, 2>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  F32Mfma<128, 2>::LDS) == hipSuccess &&
              hipFuncSetAttribute((const void *)bwd_dq_f32_mfma_kernel<64, 1>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  F32Mfma<64, 1>::LDS) == hipSuccess &&
              hipFuncSetAttribute((const void *)bwd_dq_f32_mfma_kernel<64, 2>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  F32Mfma<64, 2>::LDS) == hipSuccess &&
              hipFuncSetAttribute((const void *)bwd_dq_f32_mfma_kernel<64, 4>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  F32Mfma<64, 4>::LDS) == hipSuccess &&
              hipFuncSetAttribute((const void *)bwd_dkdv_f32_mfma_kernel<128>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  F32DkdvLds<128>::LDS) == hipSuccess &&
              hipFuncSetAttribute((const void *)bwd_dkdv_f32_mfma_kernel<64>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  F32DkdvLds<64>::LDS) == hipSuccess;
    if (!ok) {
        (void)hipGetLastError();
        return LTR_ELAUNCH;
    }
    g_dev[dev].large_lds.store(1, std::memory_order_release);
    return LTR_OK;
}

bool strides_ok(const int64_t *s, int elem_bytes) {
    const int per16 = 16 / elem_bytes;
    for (int i = 0; i < 3; i++)
        if (s[i] < 0 || (s[i] % per16) != 0) return false;
    return true;
}

int fits_i32(int64_t x) { return x >= 0 && x < (int64_t)0x7fffffff; }

// How evenly `blocks` equal blocks, one per CU at a time, fill the CUs: blocks / (rounds x CUs), 1 = no idle CU in any round.
double cu_fill(long long blocks, int cus) {
    const long long rounds = (blocks + cus - 1) / cus;
    return rounds > 0 ? (double)blocks / (double)(rounds * cus) : 0.0;
}

// compute units of the current device (the launch heuristics below count rounds of blocks over them); asked once per
// device.  Without a device (a host-only ltr_attn_plan call) the answer is that of the part this library is written for.
int device_cus() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= LTR_MAX_DEVICES) {
        (void)hipGetLastError();   // "no device" is an answer here, not an error to leave behind
        return 256;
    }
    int cus = g_dev[dev].cus.load(std::memory_order_acquire);
    if (cus <= 0) {
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return 256;
        g_dev[dev].cus.store(cus, std::memory_order_release);
    }
    return cus;
}

// One kernel launch whose own status is what is returned: hipLaunchKernel reports the submission of THIS launch, so an
// error that unrelated earlier work left in the thread's last-error slot is neither reported as ours nor cleared.
template <class Params>
int launch(const void *kernel, long long blocks, int threads, size_t lds_bytes, hipStream_t st, const Params &p) {
    void *args[] = {(void *)&p};
    return hipLaunchKernel(kernel, dim3((unsigned)blocks), dim3((unsigned)threads), args, lds_bytes, st) == hipSuccess ? LTR_OK
                                                                                                                      : LTR_ELAUNCH;
}

// Keys that the q rows [r0, r1] walk through under the causal mask: per chunk, those up to the rows' last position.
long long visible_keys(int r0, int r1, int q_split, const int *q_pos0, const ChunkDev *chunk, int n_chunks) {
    auto pos = [&](int row) { return row < q_split ? q_pos0[0] + row : q_pos0[1] + (row - q_split); };
    int hi = pos(r1);
    if (r0 < q_split && r1 >= q_split) hi = std::max(hi, pos(q_split - 1));
    long long keys = 0;
    for (int c = 0; c < n_chunks; c++) keys += std::min<long long>(std::max<long long>((long long)hi - chunk[c].pos0 + 1, 0), chunk[c].sk);
    return keys;
}

// Under a causal mask, do the q tiles of `rows` rows differ in work?  Compared are the first and the last tile: a late
// chunk of a long ring sees nearly all keys from every tile (nothing to balance), a single causal chunk 1 / n of them
// from its first tile.
bool q_tiles_uneven(int Sq, int rows, int q_split, const int *q_pos0, const ChunkDev *chunk, int n_chunks) {
    const int n = (Sq + rows - 1) / rows;
    if (n < 2) return false;
    const long long first = visible_keys(0, rows - 1, q_split, q_pos0, chunk, n_chunks);
    const long long last = visible_keys((n - 1) * rows, Sq - 1, q_split, q_pos0, chunk, n_chunks);
    return std::min(first, last) * 4 < std::max(first, last) * 3;
}

// Slots of q tiles handed to the blocks of the forward and dQ kernels.  Under a causal mask a tile's work grows with its
// rows' positions; pairing tile t with tile n - 1 - t in one block gives every block the same work (no long blocks left
// over at the end of the launch) and halves the number of blocks to start.  Only done when the tiles do differ (see
// q_tiles_uneven: paired tiles run one after the other, so fewer blocks walk through the same K / V rows at the same time)
// and while the equal blocks still fill the device's CUs evenly; otherwise one tile per slot, heaviest first, and the
// hardware's in-order dispatch balances.
int q_tile_slots(int n_qtiles, long long blocks_per_tile, bool uneven) {
    if (!uneven || n_qtiles < 2) return n_qtiles;
    const int cus = device_cus();
    const int n_slots = (n_qtiles + 1) / 2;
    const long long n = n_slots * blocks_per_tile, rounds = (n + cus - 1) / cus;
    return n * 10 >= rounds * cus * 9 ? n_slots : n_qtiles;
}

// What a forward launch looks like: rows per block, q tiles, slots (see q_tile_slots), blocks.  One function decides for
// ltr_attn_fwd and for ltr_attn_plan, so the plan a caller is shown is the launch it gets.
struct FwdPlan {
    bool wide;          // 512-row blocks (two 32-row blocks per wave, head dim 64)
    int f32_ks;         // fp32: 0 = scalar kernel, else the key shares per row group of fwd_f32_mfma_kernel
    int rows, n_qtiles, n_slots;
    long long blocks;
};
FwdPlan plan_fwd(int D, bool f32, unsigned flags, int B, int Hq, int Sq, int q_split, const int *q_pos0, const ChunkDev *chunk,
                 int n_chunks) {
    FwdPlan pl;
    pl.f32_ks = 0;
    if (f32) {
        pl.wide = false;
        if (flags & LTR_FWD_F32_SCALAR) {
            pl.rows = 64;
        } else {
            // matrix-pipe kernel: 128 rows per block, or fewer rows and the keys split over 2 / 4 waves of a row group when
            // the launch has too few rows to give every CU a block (4 key shares need the LDS that only head dim 64 leaves)
            const int cus = device_cus();
            const int max_ks = D == 64 ? 4 : 2;
            int ks = 1;
            while (ks < max_ks && (long long)((Sq + 128 / ks - 1) / (128 / ks)) * B * Hq < cus) ks *= 2;
            pl.f32_ks = ks;
            pl.rows = 128 / ks;
        }
        pl.n_qtiles = pl.n_slots = (Sq + pl.rows - 1) / pl.rows;
        pl.blocks = (long long)pl.n_qtiles * B * Hq;
        return pl;
    }
    const bool causal_ = (flags & LTR_CAUSAL) != 0;
    // query rows per block: 512 (two 32-row blocks per wave, 64-key tiles) pays at head dim 64 under the conditions of
    // the dQ kernel's 512-row blocks (see plan_bwd)
    bool wide = (flags & LTR_FWD_ROWS_512) != 0;
    if (!wide && !(flags & LTR_FWD_ROWS_256) && D == 64) {
        const int tiles512 = (Sq + 511) / 512;
        const int slots512 = q_tile_slots(tiles512, (long long)B * Hq, causal_ && q_tiles_uneven(Sq, 512, q_split, q_pos0, chunk, n_chunks));
        const long long blocks512 = (long long)slots512 * B * Hq, blocks256 = (long long)((Sq + 255) / 256) * B * Hq;
        const int cus = device_cus();
        wide = causal_ ? (Sq >= 2048 && blocks512 >= (long long)(slots512 != tiles512 ? 1 : 4) * cus)
                       : (cu_fill(blocks512, cus) * 1.07 >= cu_fill(blocks256, cus));
    }
    pl.wide = wide;
    pl.rows = wide ? 512 : 256;
    pl.n_qtiles = (Sq + pl.rows - 1) / pl.rows;
    pl.n_slots = q_tile_slots(pl.n_qtiles, (long long)B * Hq, causal_ && q_tiles_uneven(Sq, pl.rows, q_split, q_pos0, chunk, n_chunks));
    pl.blocks = (long long)pl.n_slots * B * Hq;
    return pl;
}

// The same for the two backward kernels.
struct BwdPlan {
    int f32_ks;         // fp32: 0 = scalar kernels, else the key shares per row group of bwd_dq_f32_mfma_kernel
    bool wide_kv;       // dK/dV kernel: 256 keys per block (two 32-key halves per wave, head dim 64)
    int keys_per_block;
    long long kv_tiles; // key blocks over all chunks of one (batch, kv head)
    long long kv_blocks;
    bool wide_q;        // dQ kernel: 512 rows per block
    int dq_rows, dq_qtiles, dq_slots;
    long long dq_blocks;
};
BwdPlan plan_bwd(int D, bool f32, unsigned flags, int B, int Hq, int Hkv, int Sq, int q_split, const int *q_pos0, const ChunkDev *chunk,
                 int n_chunks) {
    BwdPlan pl;
    pl.f32_ks = 0;
    if (f32) {
        pl.wide_kv = pl.wide_q = false;
        if (flags & LTR_BWD_F32_SCALAR) {
            pl.keys_per_block = 64;
            pl.dq_rows = 64;
        } else {
            // matrix-pipe kernels: 128 keys per dK/dV block; the dQ kernel sized like the fp32 forward (see plan_fwd)
            const int cus = device_cus();
            const int max_ks = D == 64 ? 4 : 2;
            int ks = 1;
            while (ks < max_ks && (long long)((Sq + 128 / ks - 1) / (128 / ks)) * B * Hq < cus) ks *= 2;
            pl.f32_ks = ks;
            pl.keys_per_block = 128;
            pl.dq_rows = 128 / ks;
        }
        pl.kv_tiles = 0;
        for (int c = 0; c < n_chunks; c++) pl.kv_tiles += (chunk[c].sk + pl.keys_per_block - 1) / pl.keys_per_block;
        pl.kv_blocks = pl.kv_tiles * B * Hkv;
        pl.dq_qtiles = pl.dq_slots = (Sq + pl.dq_rows - 1) / pl.dq_rows;
        pl.dq_blocks = (long long)pl.dq_qtiles * B * Hq;
        return pl;
    }
    const bool causal_ = (flags & LTR_CAUSAL) != 0;
    // keys per block of the dK/dV kernel: 256 (two 32-key halves per wave, about 12 % less time per key) pays at head dim 64
    // when the wider blocks fill the device's CUs about as evenly as the 128-key blocks do (equal blocks, no mask), or, under
    // a causal mask (unequal blocks), when a block walks many q tiles and there are several rounds of blocks to balance
    // with; the caller can force either size
    bool wide = (flags & LTR_DKDV_KEYS_256) != 0;
    if (!wide && !(flags & LTR_DKDV_KEYS_128) && D == 64 && !(flags & LTR_NO_DKDV)) {
        long long blocks256 = 0, blocks128 = 0;
        for (int c = 0; c < n_chunks; c++) {
            blocks256 += (chunk[c].sk + 255) / 256;
            blocks128 += (chunk[c].sk + 127) / 128;
        }
        blocks256 *= (long long)B * Hkv;
        blocks128 *= (long long)B * Hkv;
        const long long q_tiles = (long long)(Hq / Hkv) * ((Sq + 63) / 64);
        const int cus = device_cus();
        if (causal_) wide = q_tiles >= 96 && blocks256 >= 4LL * cus;
        else wide = q_tiles >= 16 && cu_fill(blocks256, cus) * 1.12 >= cu_fill(blocks128, cus);
    }
    pl.wide_kv = wide;
    pl.keys_per_block = wide ? BwdLds<64, 2>::BN : BwdLds<64, 1>::BN;
    pl.kv_tiles = 0;
    for (int c = 0; c < n_chunks; c++) pl.kv_tiles += (chunk[c].sk + pl.keys_per_block - 1) / pl.keys_per_block;
    pl.kv_blocks = pl.kv_tiles * B * Hkv;
    // query rows per block of the dQ kernel: 512 (two 32-row blocks per wave) pays at head dim 64 when the wider blocks still
    // fill the device, and under a causal mask only on sequences long enough that the diagonal does not dominate
    bool wide_q = (flags & LTR_DQ_ROWS_512) != 0;
    if (!wide_q && !(flags & LTR_DQ_ROWS_256) && D == 64 && !(flags & LTR_NO_DQ)) {
        const int tiles512 = (Sq + 511) / 512;
        const int slots512 = q_tile_slots(tiles512, (long long)B * Hq, causal_ && q_tiles_uneven(Sq, 512, q_split, q_pos0, chunk, n_chunks));
        const long long blocks512 = (long long)slots512 * B * Hq;
        const int cus = device_cus();
        // causal: equal (paired) blocks need one full round, unequal ones several rounds to balance; no mask: the wider
        // blocks (about 7 % less time per row) must fill the CUs about as evenly as the 256-row blocks
        const long long blocks256 = (long long)((Sq + 255) / 256) * B * Hq;
        wide_q = causal_ ? (Sq >= 2048 && blocks512 >= (long long)(slots512 != tiles512 ? 1 : 4) * cus)
                         : (cu_fill(blocks512, cus) * 1.07 >= cu_fill(blocks256, cus));
    }
    pl.wide_q = wide_q;
    pl.dq_rows = wide_q ? 512 : 256;
    pl.dq_qtiles = (Sq + pl.dq_rows - 1) / pl.dq_rows;
    pl.dq_slots = q_tile_slots(pl.dq_qtiles, (long long)B * Hq, causal_ && q_tiles_uneven(Sq, pl.dq_rows, q_split, q_pos0, chunk, n_chunks));
    pl.dq_blocks = (long long)pl.dq_slots * B * Hq;
    return pl;
}

// every position of the local rows lies inside the rows [pos0, pos0 + len) of a RoPE table
bool rope_table_covers(const int64_t *q_pos0, int64_t q_split, int64_t Sq, int64_t pos0, int64_t len) {
    if (len <= 0 || !fits_i32(pos0)) return false;
    if (q_split > 0 && (q_pos0[0] < pos0 || q_pos0[0] + q_split > pos0 + len)) return false;
    if (Sq > q_split && (q_pos0[1] < pos0 || q_pos0[1] + (Sq - q_split) > pos0 + len)) return false;
    return true;
}

// ------------------------------------------------------------------------------ fixed scratch
// DELTA workspace of ltr_attn_bwd_noalloc: a fixed array in device memory that belongs to the library (every device the
// library runs on holds its own copy until the process ends).  Host code never uses the array's name as an address: the
// device address of the current device's copy is looked up once per device (scratch_address) and passed to the kernels
// like any caller-owned workspace.
}  // namespace
static __device__ __align__(256) float scratch[LTR_NOALLOC_MAX_ROWS];
namespace {

int scratch_address(float **out) {
    int dev = 0;
    if (current_device(&dev)) return LTR_EDEVICE;
    float *ptr = g_dev[dev].scratch.load(std::memory_order_acquire);
    if (!ptr) {
        void *sym = nullptr;
        if (hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)) != hipSuccess || !sym) {
            (void)hipGetLastError();
            return LTR_ELAUNCH;
        }
        ptr = (float *)sym;
        g_dev[dev].scratch.store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return LTR_OK;
}

}  // namespace

extern "C" int ltr_abi_version(void) { return LTR_ABI_VERSION; }

extern "C" const char *ltr_strerror(int code) {
    switch (code) {
        case LTR_OK: return "ok";
        case LTR_EINVAL: return "invalid argument (null pointer, bad size or flag)";
        case LTR_EUNSUP: return "unsupported head dim / dtype combination";
        case LTR_EALIGN: return "pointer or stride not 16-byte aligned";
        case LTR_ELAUNCH: return "HIP launch error";
        case LTR_EDEVICE: return "current device is not gfx950";
        case LTR_ETOOBIG: return "size beyond the fixed scratch of the no-allocation entry point";
        default: return "unknown error";
    }
}

extern "C" int ltr_attn_fwd(const ltr_attn_fwd_args *a, void *stream) {
    if (!a || !a->q || !a->o || !a->lse) return LTR_EINVAL;
    if (a->B <= 0 || a->Hq <= 0 || a->Hkv <= 0 || a->Sq <= 0 || a->Hq % a->Hkv) return LTR_EINVAL;
    if (a->n_chunks < 1 || a->n_chunks > LTR_MAX_CHUNKS) return LTR_EINVAL;
    if (a->flags & ~(LTR_CAUSAL | LTR_MERGE | LTR_ROPE_Q | LTR_FWD_ROWS_256 | LTR_FWD_ROWS_512 | LTR_FWD_F32_SCALAR)) return LTR_EINVAL;
    if ((a->flags & LTR_FWD_F32_SCALAR) && a->io_dtype != LTR_F32) return LTR_EUNSUP;
    if ((a->flags & LTR_FWD_ROWS_256) && (a->flags & LTR_FWD_ROWS_512)) return LTR_EINVAL;
    if (a->D != 64 && a->D != 128) return LTR_EUNSUP;
    if (a->io_dtype != LTR_BF16 && a->io_dtype != LTR_F32) return LTR_EUNSUP;
    if (a->o_dtype != LTR_BF16 && a->o_dtype != LTR_F32) return LTR_EUNSUP;
    if (a->io_dtype == LTR_F32 && a->o_dtype != LTR_F32) return LTR_EUNSUP;
    if (!fits_i32(a->Sq) || a->q_split < 0 || a->q_split > a->Sq) return LTR_EINVAL;
    if (!fits_i32(a->q_pos0[0] + a->Sq) || !fits_i32(a->q_pos0[1] + a->Sq)) return LTR_EINVAL;
    const int eb = a->io_dtype == LTR_BF16 ? 2 : 4, ob = a->o_dtype == LTR_BF16 ? 2 : 4;
    if (!aligned16(a->q) || !aligned16(a->o) || !aligned16(a->lse)) return LTR_EALIGN;
    if (!strides_ok(a->q_stride, eb) || !strides_ok(a->k_stride, eb) || !strides_ok(a->v_stride, eb)) return LTR_EALIGN;
    // o rows are written in 4-element groups
    for (int i = 0; i < 3; i++)
        if (a->o_stride[i] < 0 || (a->o_stride[i] * ob) % 8) return LTR_EALIGN;
    FwdParams p;
    p.rope = nullptr;
    p.rope_pos0 = 0;
    p.q_rot = nullptr;
    for (int i = 0; i < 3; i++) p.qrs[i] = 0;
    if (a->flags & LTR_ROPE_Q) {
        if (a->io_dtype != LTR_BF16) return LTR_EUNSUP;
        if (!a->rope_freqs) return LTR_EINVAL;
        if (!rope_table_covers(a->q_pos0, a->q_split, a->Sq, a->rope_pos0, a->rope_len)) return LTR_EINVAL;
        if (!aligned16(a->rope_freqs) || (a->q_rot && (!aligned16(a->q_rot) || !strides_ok(a->q_rot_stride, 2)))) return LTR_EALIGN;
        p.rope = a->rope_freqs;
        p.rope_pos0 = (int)a->rope_pos0;
        p.q_rot = a->q_rot;
        for (int i = 0; i < 3; i++) p.qrs[i] = a->q_rot ? a->q_rot_stride[i] : 0;
    }
    for (int c = 0; c < a->n_chunks; c++) {
        const ltr_kv_chunk &ch = a->chunk[c];
        if (!ch.k || !ch.v || ch.sk <= 0 || !fits_i32(ch.sk) || !fits_i32(ch.pos0 + ch.sk)) return LTR_EINVAL;
        if (!aligned16(ch.k) || !aligned16(ch.v)) return LTR_EALIGN;
        // tile offsets inside a chunk are 32-bit element counts
        if ((ch.sk + 64) * a->k_stride[1] >= 0x7fffffffLL || (ch.sk + 64) * a->v_stride[1] >= 0x7fffffffLL) return LTR_EUNSUP;
        p.chunk[c].k = ch.k;
        p.chunk[c].v = ch.v;
        p.chunk[c].dk = nullptr;
        p.chunk[c].dv = nullptr;
        p.chunk[c].sk = (int)ch.sk;
        p.chunk[c].pos0 = (int)ch.pos0;
    }
    int rc = check_device();
    if (rc) return rc;
    p.q = a->q;
    p.o = a->o;
    p.lse = a->lse;
    p.B = a->B;
    p.Hq = a->Hq;
    p.Hkv = a->Hkv;
    p.n_rep = a->Hq / a->Hkv;
    p.Sq = (int)a->Sq;
    for (int i = 0; i < 3; i++) {
        p.qs[i] = a->q_stride[i];
        p.os[i] = a->o_stride[i];
        p.ks[i] = a->k_stride[i];
        p.vs[i] = a->v_stride[i];
    }
    p.q_pos0[0] = (int)a->q_pos0[0];
    p.q_pos0[1] = (int)a->q_pos0[1];
    p.q_split = (int)a->q_split;
    p.scale = a->scale;
    p.flags = a->flags & (LTR_CAUSAL | LTR_MERGE | LTR_ROPE_Q);
    p.o_f32 = a->o_dtype == LTR_F32;
    p.n_chunks = a->n_chunks;
    hipStream_t st = (hipStream_t)stream;
    if ((a->flags & LTR_FWD_ROWS_512) && (a->D != 64 || a->io_dtype != LTR_BF16)) return LTR_EUNSUP;
    const FwdPlan pl = plan_fwd(a->D, a->io_dtype == LTR_F32, a->flags, p.B, p.Hq, p.Sq, p.q_split, p.q_pos0, p.chunk, p.n_chunks);
    if (pl.blocks > 0x7fffffffLL) return LTR_EINVAL;
    p.n_qtiles = pl.n_qtiles;
    p.n_slots = pl.n_slots;
    if (a->io_dtype == LTR_BF16) {
        rc = enable_large_lds();
        if (rc) return rc;
        if (a->D == 128) return launch((const void *)fwd_bf16_kernel<128, 1>, pl.blocks, 512, fwd_lds_bytes<128>(), st, p);
        if (pl.wide) return launch((const void *)fwd_bf16_kernel<64, 2>, pl.blocks, 512, fwd_lds_bytes<64, 2>(), st, p);
        return launch((const void *)fwd_bf16_kernel<64, 1>, pl.blocks, 512, fwd_lds_bytes<64>(), st, p);
    }
    if (pl.f32_ks) {   // fp32 on the matrix pipe; the chunk offsets of its LDS-direct loads are 64-bit, nothing more to check
        rc = enable_large_lds();
        if (rc) return rc;
        if (a->D == 128) {
            if (pl.f32_ks == 1) return launch((const void *)fwd_f32_mfma_kernel<128, 1>, pl.blocks, 256, F32Mfma<128, 1>::LDS, st, p);
            return launch((const void *)fwd_f32_mfma_kernel<128, 2>, pl.blocks, 256, F32Mfma<128, 2>::LDS, st, p);
        }
        if (pl.f32_ks == 1) return launch((const void *)fwd_f32_mfma_kernel<64, 1>, pl.blocks, 256, F32Mfma<64, 1>::LDS, st, p);
        if (pl.f32_ks == 2) return launch((const void *)fwd_f32_mfma_kernel<64, 2>, pl.blocks, 256, F32Mfma<64, 2>::LDS, st, p);
        return launch((const void *)fwd_f32_mfma_kernel<64, 4>, pl.blocks, 256, F32Mfma<64, 4>::LDS, st, p);
    }
    if (a->D == 128) return launch((const void *)fwd_f32_kernel<128>, pl.blocks, 64, 0, st, p);
    return launch((const void *)fwd_f32_kernel<64>, pl.blocks, 64, 0, st, p);
}

extern "C" int ltr_attn_bwd_delta(const ltr_attn_delta_args *a, void *stream) {
    if (!a || !a->o || !a->d_o || !a->delta) return LTR_EINVAL;
    if (a->B <= 0 || a->Hq <= 0 || a->Sq <= 0 || !fits_i32(a->Sq)) return LTR_EINVAL;
    if (a->D != 64 && a->D != 128) return LTR_EUNSUP;
    if ((a->o_dtype != LTR_BF16 && a->o_dtype != LTR_F32) || (a->do_dtype != LTR_BF16 && a->do_dtype != LTR_F32))
        return LTR_EUNSUP;
    for (int i = 0; i < 3; i++)
        if (a->o_stride[i] < 0 || a->do_stride[i] < 0) return LTR_EINVAL;
    int rc = check_device();
    if (rc) return rc;
    DeltaParams p;
    p.o = a->o;
    p.d_o = a->d_o;
    p.delta = a->delta;
    p.B = a->B;
    p.Hq = a->Hq;
    p.D = a->D;
    p.Sq = (int)a->Sq;
    for (int i = 0; i < 3; i++) {
        p.os[i] = a->o_stride[i];
        p.dos[i] = a->do_stride[i];
    }
    p.o_f32 = a->o_dtype == LTR_F32;
    p.do_f32 = a->do_dtype == LTR_F32;
    const long long nthreads = (long long)p.B * p.Hq * p.Sq * 16;
    const long long nblk = (nthreads + 255) / 256;
    if (nblk > 0x7fffffffLL) return LTR_EINVAL;
    return launch((const void *)delta_kernel, nblk, 256, 0, (hipStream_t)stream, p);
}

namespace {
// ltr_attn_bwd (DELTA is the caller's buffer) and ltr_attn_bwd_noalloc (use_scratch: DELTA lives in the library's fixed
// scratch array; flags already carry LTR_DELTA_FROM_O)
int bwd_launch(const ltr_attn_bwd_args *a, unsigned flags, bool use_scratch, void *stream) {
    float *delta = use_scratch ? nullptr : a->delta;
    if (!a->q || !a->d_o || !a->lse || (!use_scratch && !delta)) return LTR_EINVAL;
    const bool do_dq = !(flags & LTR_NO_DQ), do_dkdv = !(flags & LTR_NO_DKDV);
    if (do_dq && !a->dq) return LTR_EINVAL;
    if (a->B <= 0 || a->Hq <= 0 || a->Hkv <= 0 || a->Sq <= 0 || a->Hq % a->Hkv) return LTR_EINVAL;
    if (a->n_chunks < 1 || a->n_chunks > LTR_MAX_CHUNKS) return LTR_EINVAL;
    if (flags & ~(LTR_CAUSAL | LTR_NO_DQ | LTR_NO_DKDV | LTR_DQ_BF16 | LTR_DELTA_FROM_O | LTR_DKDV_BF16 | LTR_ROPE_DQ | LTR_DKDV_KEYS_128 |
                  LTR_DKDV_KEYS_256 | LTR_DQ_ROWS_256 | LTR_DQ_ROWS_512 | LTR_BWD_F32_SCALAR))
        return LTR_EINVAL;
    if ((flags & LTR_BWD_F32_SCALAR) && a->io_dtype != LTR_F32) return LTR_EUNSUP;
    if ((flags & LTR_DKDV_KEYS_128) && (flags & LTR_DKDV_KEYS_256)) return LTR_EINVAL;
    if ((flags & LTR_DQ_ROWS_256) && (flags & LTR_DQ_ROWS_512)) return LTR_EINVAL;
    const bool fused_delta = flags & LTR_DELTA_FROM_O;
    if (fused_delta && (!do_dq || !a->o)) return LTR_EINVAL;
    if (a->D != 64 && a->D != 128) return LTR_EUNSUP;
    if (a->io_dtype != LTR_BF16 && a->io_dtype != LTR_F32) return LTR_EUNSUP;
    const bool f32 = a->io_dtype == LTR_F32;
    if (f32 && (flags & (LTR_DQ_BF16 | LTR_DELTA_FROM_O | LTR_DKDV_BF16 | LTR_ROPE_DQ | LTR_DKDV_KEYS_256 | LTR_DQ_ROWS_512)))
        return LTR_EUNSUP;   // bf16 conveniences and kernels only
    const int gb = (flags & LTR_DKDV_BF16) ? 2 : 4;   // bytes per dK / dV element
    const int eb = f32 ? 4 : 2;
    if (!fits_i32(a->Sq) || a->q_split < 0 || a->q_split > a->Sq) return LTR_EINVAL;
    if (!fits_i32(a->q_pos0[0] + a->Sq) || !fits_i32(a->q_pos0[1] + a->Sq)) return LTR_EINVAL;
    if (!aligned16(a->q) || !aligned16(a->d_o) || (do_dq && !aligned16(a->dq))) return LTR_EALIGN;
    if (!strides_ok(a->q_stride, eb) || !strides_ok(a->do_stride, eb) || !strides_ok(a->k_stride, eb) ||
        !strides_ok(a->v_stride, eb) || !strides_ok(a->dk_stride, gb) || !strides_ok(a->dv_stride, gb))
        return LTR_EALIGN;
    for (int i = 0; i < 3; i++)
        if (a->dq_stride[i] < 0) return LTR_EINVAL;
    if (do_dq && !strides_ok(a->dq_stride, (flags & LTR_DQ_BF16) ? 2 : 4)) return LTR_EALIGN;
    if (fused_delta && (!aligned16(a->o) || !strides_ok(a->o_stride, 2))) return LTR_EALIGN;
    if (fused_delta && (a->Sq + 64) * a->o_stride[1] >= 0x7fffffffLL) return LTR_EUNSUP;
    if ((a->Sq + 63) / 64 > BwdLds<128, 1>::MAX_QTILES) return LTR_EUNSUP;       // q tile lists live in LDS
    if ((a->Sq + 64) * a->q_stride[1] >= 0x7fffffffLL || (a->Sq + 64) * a->do_stride[1] >= 0x7fffffffLL) return LTR_EUNSUP;
    BwdParams p;
    p.rope = nullptr;
    p.rope_pos0 = 0;
    if (flags & LTR_ROPE_DQ) {
        if (!do_dq || !a->rope_freqs) return LTR_EINVAL;
        if (!rope_table_covers(a->q_pos0, a->q_split, a->Sq, a->rope_pos0, a->rope_len)) return LTR_EINVAL;
        if (!aligned16(a->rope_freqs)) return LTR_EALIGN;
        p.rope = a->rope_freqs;
        p.rope_pos0 = (int)a->rope_pos0;
    }
    if ((flags & LTR_DKDV_KEYS_256) && (a->D != 64 || f32)) return LTR_EUNSUP;
    if ((flags & LTR_DQ_ROWS_512) && a->D != 64) return LTR_EUNSUP;
    for (int c = 0; c < a->n_chunks; c++) {
        const ltr_kv_chunk &ch = a->chunk[c];
        if (!ch.k || !ch.v || ch.sk <= 0 || !fits_i32(ch.sk) || !fits_i32(ch.pos0 + ch.sk)) return LTR_EINVAL;
        if (do_dkdv && (!ch.dk || !ch.dv)) return LTR_EINVAL;
        if ((ch.sk + 64) * a->k_stride[1] >= 0x7fffffffLL || (ch.sk + 64) * a->v_stride[1] >= 0x7fffffffLL) return LTR_EUNSUP;
        if (!aligned16(ch.k) || !aligned16(ch.v)) return LTR_EALIGN;
        if (do_dkdv && (!aligned16(ch.dk) || !aligned16(ch.dv))) return LTR_EALIGN;
        p.chunk[c].k = ch.k;
        p.chunk[c].v = ch.v;
        p.chunk[c].dk = (float *)ch.dk;
        p.chunk[c].dv = (float *)ch.dv;
        p.chunk[c].sk = (int)ch.sk;
        p.chunk[c].pos0 = (int)ch.pos0;
    }
    int rc = check_device();
    if (rc) return rc;
    if (use_scratch) {
        rc = scratch_address(&delta);
        if (rc) return rc;
    }
    p.q = a->q;
    p.d_o = a->d_o;
    p.lse = a->lse;
    p.delta = delta;
    p.o = a->o;
    for (int i = 0; i < 3; i++) p.os_[i] = fused_delta ? a->o_stride[i] : 0;
    p.dq = a->dq;
    p.B = a->B;
    p.Hq = a->Hq;
    p.Hkv = a->Hkv;
    p.n_rep = a->Hq / a->Hkv;
    p.Sq = (int)a->Sq;
    p.n_qtiles = (p.Sq + 63) / 64;
    for (int i = 0; i < 3; i++) {
        p.qs[i] = a->q_stride[i];
        p.dos[i] = a->do_stride[i];
        p.dqs[i] = a->dq_stride[i];
        p.ks[i] = a->k_stride[i];
        p.vs[i] = a->v_stride[i];
        p.dks[i] = a->dk_stride[i];
        p.dvs[i] = a->dv_stride[i];
    }
    p.q_pos0[0] = (int)a->q_pos0[0];
    p.q_pos0[1] = (int)a->q_pos0[1];
    p.q_split = (int)a->q_split;
    p.scale = a->scale;
    p.flags = flags;
    p.n_chunks = a->n_chunks;
    const BwdPlan pl = plan_bwd(a->D, f32, flags, p.B, p.Hq, p.Hkv, p.Sq, p.q_split, p.q_pos0, p.chunk, p.n_chunks);
    if (pl.kv_blocks > 0x7fffffffLL || pl.dq_blocks > 0x7fffffffLL) return LTR_EINVAL;
    p.tiles_total = (int)pl.kv_tiles;
    p.n_slots = pl.dq_slots;
    hipStream_t st = (hipStream_t)stream;
    if (f32 && pl.f32_ks) {   // fp32 on the matrix pipe
        rc = enable_large_lds();
        if (rc) return rc;
        if (do_dq) {
            if (a->D == 128)
                rc = pl.f32_ks == 1 ? launch((const void *)bwd_dq_f32_mfma_kernel<128, 1>, pl.dq_blocks, 256, F32Mfma<128, 1>::LDS, st, p)
                                    : launch((const void *)bwd_dq_f32_mfma_kernel<128, 2>, pl.dq_blocks, 256, F32Mfma<128, 2>::LDS, st, p);
            else
                rc = pl.f32_ks == 1   ? launch((const void *)bwd_dq_f32_mfma_kernel<64, 1>, pl.dq_blocks, 256, F32Mfma<64, 1>::LDS, st, p)
                     : pl.f32_ks == 2 ? launch((const void *)bwd_dq_f32_mfma_kernel<64, 2>, pl.dq_blocks, 256, F32Mfma<64, 2>::LDS, st, p)
                                      : launch((const void *)bwd_dq_f32_mfma_kernel<64, 4>, pl.dq_blocks, 256, F32Mfma<64, 4>::LDS, st, p);
            if (rc) return rc;
        }
        if (do_dkdv)
            rc = a->D == 128 ? launch((const void *)bwd_dkdv_f32_mfma_kernel<128>, pl.kv_blocks, 256, F32DkdvLds<128>::LDS, st, p)
                             : launch((const void *)bwd_dkdv_f32_mfma_kernel<64>, pl.kv_blocks, 256, F32DkdvLds<64>::LDS, st, p);
        return rc;
    }
    if (f32) {
        if (do_dq) {
            rc = a->D == 128 ? launch((const void *)bwd_dq_f32_kernel<128>, pl.dq_blocks, 64, 0, st, p)
                             : launch((const void *)bwd_dq_f32_kernel<64>, pl.dq_blocks, 64, 0, st, p);
            if (rc) return rc;
        }
        if (do_dkdv) {
            rc = a->D == 128 ? launch((const void *)bwd_dkdv_f32_kernel<128, false>, pl.kv_blocks, 64, 0, st, p)
                             : launch((const void *)bwd_dkdv_f32_kernel<64, false>, pl.kv_blocks, 64, 0, st, p);
            if (rc) return rc;
            rc = a->D == 128 ? launch((const void *)bwd_dkdv_f32_kernel<128, true>, pl.kv_blocks, 64, 0, st, p)
                             : launch((const void *)bwd_dkdv_f32_kernel<64, true>, pl.kv_blocks, 64, 0, st, p);
        }
        return rc;
    }
    rc = enable_large_lds();
    if (rc) return rc;
    // the dQ kernel goes first: with LTR_DELTA_FROM_O it produces the DELTA that the dK/dV kernel reads
    if (do_dq) {
        if (a->D == 128) rc = launch((const void *)bwd_dq_kernel<128, 1>, pl.dq_blocks, 512, dq_lds_bytes<128>(), st, p);
        else if (pl.wide_q) rc = launch((const void *)bwd_dq_kernel<64, 2>, pl.dq_blocks, 512, dq_lds_bytes<64>(), st, p);
        else rc = launch((const void *)bwd_dq_kernel<64, 1>, pl.dq_blocks, 512, dq_lds_bytes<64>(), st, p);
        if (rc) return rc;
    }
    if (do_dkdv) {
        // A block of the dK/dV kernel owns 128 keys and loops over the query tiles that see them: under a causal mask its
        // work falls with the keys' position.  The blocks of one (batch, kv head) are handed out in the order of the chunk
        // table, so the table of THIS kernel is sorted by position: the longest blocks start first and the short ones fill
        // the tail (the sums inside a block do not depend on the table's order).
        if (flags & LTR_CAUSAL)
            std::stable_sort(p.chunk, p.chunk + p.n_chunks, [](const ChunkDev &x, const ChunkDev &y) { return x.pos0 < y.pos0; });
        if (a->D == 128) rc = launch((const void *)bwd_dkdv_kernel<128, 1>, pl.kv_blocks, BwdLds<128, 1>::NT, BwdLds<128, 1>::TOTAL, st, p);
        else if (pl.wide_kv) rc = launch((const void *)bwd_dkdv_kernel<64, 2>, pl.kv_blocks, BwdLds<64, 2>::NT, BwdLds<64, 2>::TOTAL, st, p);
        else rc = launch((const void *)bwd_dkdv_kernel<64, 1>, pl.kv_blocks, BwdLds<64, 1>::NT, BwdLds<64, 1>::TOTAL, st, p);
    }
    return rc;
}
}  // namespace

extern "C" int ltr_attn_bwd(const ltr_attn_bwd_args *a, void *stream) {
    if (!a) return LTR_EINVAL;
    return bwd_launch(a, a->flags, false, stream);
}

// Host-only: nothing is enqueued, no pointer is read.
extern "C" int ltr_attn_plan(const ltr_attn_bwd_args *a, ltr_attn_plan_t *out) {
    if (!a || !out) return LTR_EINVAL;
    if (a->B <= 0 || a->Hq <= 0 || a->Hkv <= 0 || a->Sq <= 0 || a->Hq % a->Hkv) return LTR_EINVAL;
    if (a->n_chunks < 1 || a->n_chunks > LTR_MAX_CHUNKS) return LTR_EINVAL;
    if (a->D != 64 && a->D != 128) return LTR_EUNSUP;
    if (a->io_dtype != LTR_BF16 && a->io_dtype != LTR_F32) return LTR_EUNSUP;
    if (!fits_i32(a->Sq) || a->q_split < 0 || a->q_split > a->Sq) return LTR_EINVAL;
    if (!fits_i32(a->q_pos0[0] + a->Sq) || !fits_i32(a->q_pos0[1] + a->Sq)) return LTR_EINVAL;
    const unsigned flags = a->flags;
    if ((flags & LTR_DKDV_KEYS_128) && (flags & LTR_DKDV_KEYS_256)) return LTR_EINVAL;
    if ((flags & LTR_DQ_ROWS_256) && (flags & LTR_DQ_ROWS_512)) return LTR_EINVAL;
    if ((flags & LTR_FWD_ROWS_256) && (flags & LTR_FWD_ROWS_512)) return LTR_EINVAL;
    const bool f32 = a->io_dtype == LTR_F32;
    if ((flags & (LTR_DKDV_KEYS_256 | LTR_DQ_ROWS_512 | LTR_FWD_ROWS_512)) && (a->D != 64 || f32)) return LTR_EUNSUP;
    if ((flags & (LTR_FWD_F32_SCALAR | LTR_BWD_F32_SCALAR)) && !f32) return LTR_EUNSUP;
    ChunkDev chunk[LTR_MAX_CHUNKS];
    for (int c = 0; c < a->n_chunks; c++) {
        const ltr_kv_chunk &ch = a->chunk[c];
        if (ch.sk <= 0 || !fits_i32(ch.sk) || !fits_i32(ch.pos0 + ch.sk)) return LTR_EINVAL;
        chunk[c].k = chunk[c].v = nullptr;
        chunk[c].dk = chunk[c].dv = nullptr;
        chunk[c].sk = (int)ch.sk;
        chunk[c].pos0 = (int)ch.pos0;
    }
    const int q_pos0[2] = {(int)a->q_pos0[0], (int)a->q_pos0[1]};
    const FwdPlan f = plan_fwd(a->D, f32, flags, a->B, a->Hq, (int)a->Sq, (int)a->q_split, q_pos0, chunk, a->n_chunks);
    const BwdPlan b = plan_bwd(a->D, f32, flags, a->B, a->Hq, a->Hkv, (int)a->Sq, (int)a->q_split, q_pos0, chunk, a->n_chunks);
    out->compute_units = device_cus();
    out->fwd_rows = f.rows;
    out->fwd_paired = f.n_slots != f.n_qtiles;
    out->fwd_blocks = f.blocks;
    out->dq_rows = b.dq_rows;
    out->dq_paired = b.dq_slots != b.dq_qtiles;
    out->dq_blocks = b.dq_blocks;
    out->dkdv_keys = b.keys_per_block;
    out->dkdv_blocks = b.kv_blocks;
    if (f32) {
        if (f.f32_ks) snprintf(out->fwd_kernel, sizeof(out->fwd_kernel), "fwd_f32_mfma_kernel<%d, %d>", a->D, f.f32_ks);
        else snprintf(out->fwd_kernel, sizeof(out->fwd_kernel), "fwd_f32_kernel<%d>", a->D);
        if (b.f32_ks) {
            snprintf(out->dq_kernel, sizeof(out->dq_kernel), "bwd_dq_f32_mfma_kernel<%d, %d>", a->D, b.f32_ks);
            snprintf(out->dkdv_kernel, sizeof(out->dkdv_kernel), "bwd_dkdv_f32_mfma_kernel<%d>", a->D);
        } else {
            snprintf(out->dq_kernel, sizeof(out->dq_kernel), "bwd_dq_f32_kernel<%d>", a->D);
            snprintf(out->dkdv_kernel, sizeof(out->dkdv_kernel), "bwd_dkdv_f32_kernel<%d, *>", a->D);
        }
    } else {
        snprintf(out->fwd_kernel, sizeof(out->fwd_kernel), "fwd_bf16_kernel<%d, %d>", a->D, f.wide ? 2 : 1);
        snprintf(out->dq_kernel, sizeof(out->dq_kernel), "bwd_dq_kernel<%d, %d>", a->D, b.wide_q ? 2 : 1);
        snprintf(out->dkdv_kernel, sizeof(out->dkdv_kernel), "bwd_dkdv_kernel<%d, %d>", a->D, b.wide_kv ? 2 : 1);
    }
    return LTR_OK;
}

extern "C" int ltr_attn_bwd_noalloc(const ltr_attn_bwd_args *a, void *stream) {
    if (!a) return LTR_EINVAL;
    if (a->io_dtype != LTR_BF16) return LTR_EUNSUP;                 // DELTA comes from the bf16 forward output
    if (a->flags & LTR_NO_DQ) return LTR_EINVAL;                    // the dQ kernel is the one that fills DELTA
    if (a->B <= 0 || a->Hq <= 0 || a->Sq <= 0) return LTR_EINVAL;
    if (a->Sq > LTR_NOALLOC_MAX_ROWS || (long long)a->B * a->Hq > LTR_NOALLOC_MAX_ROWS ||
        (long long)a->B * a->Hq * a->Sq > LTR_NOALLOC_MAX_ROWS)
        return LTR_ETOOBIG;
    return bwd_launch(a, a->flags | LTR_DELTA_FROM_O, true, stream);
}

extern "C" int ltr_cast_f32_to_bf16(const float *src, void *dst, int64_t n, void *stream) {
    if (!src || !dst || n < 0) return LTR_EINVAL;
    if (n == 0) return LTR_OK;
    if (!aligned16(src) || ((uintptr_t)dst & 7)) return LTR_EALIGN;
    int rc = check_device();
    if (rc) return rc;
    const long long nblk = (n / 4 + 256) / 256;
    if (nblk > 0x7fffffffLL) return LTR_EINVAL;
    __bf16 *dst16 = (__bf16 *)dst;
    long long n64 = n;
    void *args[] = {(void *)&src, (void *)&dst16, (void *)&n64};
    return hipLaunchKernel((const void *)cast_kernel, dim3((unsigned)nblk), dim3(256), args, 0, (hipStream_t)stream) == hipSuccess
               ? LTR_OK
               : LTR_ELAUNCH;
}
