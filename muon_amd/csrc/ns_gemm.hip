// Grouped bf16 MFMA GEMM for the Newton-Schulz iteration on gfx950 (CDNA4).
//
// Every product of the iteration (muon.py:285-287) is computed by one kernel as
//     acc[i][j] = sum_k P[i][k] * Q[j][k]          (both operands row-major along k), or
//     acc[i][j] = sum_k P[i][k] * Q[k][j]          (second operand k-major):
//     A  = X X^T                P = Q = X            (rows of X)
//     A A (A symmetric)         P = A or c*A, Q = A  ((A A)[i][j] = sum_k A[i][k] A[j][k])
//     B X                       P = B, Q = X itself, k-major (no transposed copy of X is kept:
//                               the fragments of Q come out of LDS through transposing reads)
// The epilogue fuses the polynomial terms (b*A + c*A*A, a*X + B*X), writes the tile and, for a
// symmetric result, its mirror image, and optionally a scaled copy (c*A).  Symmetric results only
// compute tiles on or above the diagonal.  The update writes X' into a second buffer (every tile of
// a column block reads all rows of X, so X cannot be overwritten in place).
//
// A launch covers a job list of output tiles drawn from many matrices; a workgroup computes one
// BM x BN tile at a time and walks its share of the list:
//   * buffer_load_dwordx4 ... lds streams the operand tiles straight into an LDS ring (no register
//     staging) in k-blocks of BK = 64, so every request is a full 128-byte line of one operand
//     row; the ring keeps a block and a half in flight while the current one is multiplied;
//   * LDS rows are 128 bytes (8 chunks of 16 bytes); chunk c of row r sits at position
//     c ^ ((r >> 1) & 7), so the 1 KiB-contiguous DMA writes and the ds_read_b128 fragment reads
//     are both bank-conflict free (a k-major operand: rows of 2 BN bytes, 64-byte blocks
//     XOR-swizzled with row & 3, read with ds_read_b64_tr_b16);
//   * each wave owns a 128 x 64 (or 64 x 64) sub-tile as 32 x 32 v_mfma_f32_32x32x16_bf16 tiles
//     with fp32 accumulation;
//   * the epilogue moves tiles between the "lane owns a column" accumulator layout and the
//     "lane owns a row" layout with two MFMAs against a permuted identity, so that the addend is
//     read and the outputs are written with wide, coalesced accesses staged through wave-private
//     LDS.
#include <stdlib.h>

#include "common.h"

#include <string.h>

#include <atomic>
#include <mutex>
#include <vector>

namespace muon_amd {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Accesses through the global (not flat) address space: pointers fetched from a descriptor are
// generic to the compiler, and a flat access would also count against the LDS wait counter.
__device__ __forceinline__ u32x2 gload8(const uint16_t* p) {
    return *(const __attribute__((address_space(1))) u32x2*)(p);
}
// STREAM: non-temporal hint.  The outputs of the large tile class are hundreds of megabytes that
// the next launch reads long after this XCD's L2 has turned over; keeping them out of the way of
// the operand panels measured +0.5 % on the Llama step (and a loss for GPT-2-size matrices, whose
// outputs the next launch does find in L2, so the small class stores normally).
template <bool STREAM>
__device__ __forceinline__ void gstore16(uint16_t* p, u32x4 v) {
    if constexpr (STREAM) __builtin_nontemporal_store(v, (__attribute__((address_space(1))) u32x4*)(p));
    else *(__attribute__((address_space(1))) u32x4*)(p) = v;
}

constexpr int BK = 64;   // k extent of one ring stage (128 bytes per LDS row)
constexpr int ROW_BYTES = BK * 2;

// One wave-wide 16-byte-per-lane load from global memory straight into LDS at
// lds_addr + lane*16 (lds_addr wave-uniform): buffer_load_dwordx4 ... lds, the operand addressed as
// resource (base pointer) + per-lane byte offset + wave-uniform byte offset.  Issued through inline
// assembly so that the compiler's wait-count insertion does not serialise the ring; completion is
// awaited explicitly with s_waitcnt vmcnt(n) before the workgroup barrier that publishes a stage.
// The buffer form keeps the per-lane address in one register and the k-block offset in a scalar one
// (global_load_lds_dwordx4 needs a 64-bit address per lane): measured 1.3 % faster on the 256 x 256
// class, equal on the 128 x 128 class.
// rsrc: {base[31:0], base[47:32] (stride 0), number of bytes addressable, format word}.
__device__ __forceinline__ u32x4 dma_resource(const void* base) {
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    return u32x4{static_cast<uint32_t>(a), static_cast<uint32_t>(a >> 32) & 0xffffu, 0xffffffffu, 0x00020000u};
}
__device__ __forceinline__ void dma16(u32x4 rsrc, uint32_t voff, uint32_t soff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds\n"
                 :: "v"(voff), "s"(rsrc), "s"(soff), "s"(lds_addr) : "memory", "m0");
}
// s_waitcnt vmcnt(n) only (expcnt / lgkmcnt left unconstrained); n < 64 (bits 3:0 and 15:14).
#define NS_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))

// Wait until at most min(n, H) half-stages (DPH DMA instructions each) of this wave are pending.
template <int DPH, int H>
struct WaitHalves {
    static __device__ __forceinline__ void run(int n) {
        if (n >= H) NS_WAIT_VMCNT(H * DPH);
        else WaitHalves<DPH, H - 1>::run(n);
    }
};
template <int DPH>
struct WaitHalves<DPH, 0> {
    static __device__ __forceinline__ void run(int) { NS_WAIT_VMCNT(0); }
};

// Fragment reads of the main loop: N ds_read_b128 from LDS byte address addr + i * 32 rows, issued
// through inline assembly so that the waits for them can be placed by hand (wait_frags).
template <int N, int I = 0>
struct FragLoad {
    static __device__ __forceinline__ void run(u32x4 (&f)[N], uint32_t addr) {
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f[I]) : "v"(addr), "n"(I * 32 * ROW_BYTES));
        if constexpr (I + 1 < N) FragLoad<N, I + 1>::run(f, addr);
    }
};
// The same for an operand that lies k-major in LDS (row = k, the tile's columns along the row: X
// itself as the second operand of B X): ds_read_b64_tr_b16 takes, in every group of 16 lanes, from
// lane 4r + c the address of columns 4c .. 4c+3 of row r of a 4 x 16 block and hands lane j the four
// rows of column j.  With lanes 0..15 / 16..31 on columns 0..15 / 16..31 of rows 0..3 and lanes 32..63
// on rows 8..11, two such reads (rows +0 and +4) leave lane l with k = 8 (l / 32) .. + 7 of column
// l % 32: exactly the second operand of v_mfma_f32_32x32x16_bf16 (checked on the device).
// f[2 i], f[2 i + 1]: the two halves of fragment i; addr[i]: its per-lane LDS byte address (the
// 64-byte column blocks of a row are XOR-swizzled with row & 3, so it depends on i).
template <int N, int ROWQ, int I = 0>
struct FragLoadTr {
    static __device__ __forceinline__ void run(u32x2 (&f)[2 * N], const uint32_t (&addr)[N], uint32_t base) {
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:0" : "=v"(f[2 * I]) : "v"(addr[I] + base));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(f[2 * I + 1]) : "v"(addr[I] + base), "n"(4 * ROWQ));
        if constexpr (I + 1 < N) FragLoadTr<N, ROWQ, I + 1>::run(f, addr, base);
    }
};

// s_waitcnt lgkmcnt(CNT), tied to the fragment registers the following MFMAs read: the compiler
// sees them redefined here and cannot move a use above the wait.
template <int CNT, int TM, int TN>
__device__ __forceinline__ void wait_frags(u32x4 (&a)[TM], u32x4 (&b)[TN]) {
    static_assert(CNT >= 0 && CNT < 16, "lgkmcnt is a 4-bit counter");
    if constexpr (TM == 4 && TN == 2)
        asm volatile("s_waitcnt lgkmcnt(%6)" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]) : "n"(CNT));
    else if constexpr (TM == 2 && TN == 2)
        asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(a[0]), "+v"(a[1]), "+v"(b[0]), "+v"(b[1]) : "n"(CNT));
    else
        static_assert(TM == 2 && TN == 2, "wait_frags: add the operand list of this wave tile");
}
template <int CNT, int TM, int TN2>
__device__ __forceinline__ void wait_frags_tr(u32x4 (&a)[TM], u32x2 (&b)[TN2]) {
    static_assert(CNT >= 0 && CNT < 16, "lgkmcnt is a 4-bit counter");
    if constexpr (TM == 4 && TN2 == 4)
        asm volatile("s_waitcnt lgkmcnt(%8)" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]),
                     "+v"(b[2]), "+v"(b[3]) : "n"(CNT));
    else if constexpr (TM == 2 && TN2 == 4)
        asm volatile("s_waitcnt lgkmcnt(%6)" : "+v"(a[0]), "+v"(a[1]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]) : "n"(CNT));
    else
        static_assert(TM == 2 && TN2 == 4, "wait_frags_tr: add the operand list of this wave tile");
}

// ---------------------------------------------------------------------------------------------
// Epilogue helpers
// ---------------------------------------------------------------------------------------------
// out = V^T for a 32 x 32 tile of bf16-representable values held in accumulator layout (lane =
// column l%32, register 4q+e = row 8q + 4(l/32) + e).  V goes in as the A operand; id0/id1 are the
// B operands with B[slot][j] = (row(slot) == j), where slot (g, t) of k-block h carries tile row
// 16h + 8(t/4) + 4g + t%4 -- exactly the rows registers 8h .. 8h+7 hold.  bf16 x 1.0 products and
// sums of a single non-zero term are exact in the fp32 accumulator.
__device__ __forceinline__ f32x16 tile_transpose_bf16(const float (&v)[16], bf16x8 id0, bf16x8 id1) {
    bf16x8 f0, f1;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        f0[t] = static_cast<__bf16>(v[t]);
        f1[t] = static_cast<__bf16>(v[8 + t]);
    }
    f32x16 z;
#pragma unroll
    for (int i = 0; i < 16; ++i) z[i] = 0.f;
    z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f0, id0, z, 0, 0, 0);
    z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f1, id1, z, 0, 0, 0);
    return z;
}

// The same for a tile already packed two bf16 per register (p[k] = values 2k, 2k+1).
__device__ __forceinline__ f32x16 tile_transpose_packed(const uint32_t (&p)[8], bf16x8 id0, bf16x8 id1) {
    const bf16x8 f0 = __builtin_bit_cast(bf16x8, u32x4{p[0], p[1], p[2], p[3]});
    const bf16x8 f1 = __builtin_bit_cast(bf16x8, u32x4{p[4], p[5], p[6], p[7]});
    f32x16 z;
#pragma unroll
    for (int i = 0; i < 16; ++i) z[i] = 0.f;
    z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f0, id0, z, 0, 0, 0);
    z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f1, id1, z, 0, 0, 0);
    return z;
}

// bf16(gamma * x) for 8 packed bf16 values.
__device__ __forceinline__ u32x4 scale_bf16x8(u32x4 v, float gamma) {
    u32x4 r;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float lo = gamma * __uint_as_float(v[k] << 16);
        const float hi = gamma * __uint_as_float(v[k] & 0xffff0000u);
        r[k] = pack2bf(lo, hi);
    }
    return r;
}

// The parameter step fused into the epilogue of the last update product (muon.py:14, 98-99):
//     update = bf16(o * scale);  param <- param * wd_factor - lr * update;  out <- update
// for 8 consecutive elements of parameter row `prow` starting at column `pcol`, o packed as bf16.
// The arithmetic is apply_kernel's (elementwise.hip), in the storage type of the parameter.
struct ApplyArgs {
    const MuonMatDesc* mat;
    float neg_lr, wd_factor;
    bool vec_ok;          // 16-byte accesses are possible: cols % 8 == 0 and aligned base pointers
};

__device__ __forceinline__ void apply_chunk8(const ApplyArgs& ap, int prow, int pcol, u32x4 v) {
    const MuonMatDesc& m = *ap.mat;
    if (prow >= m.rows || pcol >= m.cols) return;          // padding rows / columns of the tile grid
    float us[8];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        us[2 * k] = round_bf(__uint_as_float(v[k] << 16) * m.scale);
        us[2 * k + 1] = round_bf(__uint_as_float(v[k] & 0xffff0000u) * m.scale);
    }
    const int64_t e = static_cast<int64_t>(prow) * m.cols + pcol;
    const bool full = ap.vec_ok && pcol + 8 <= m.cols;
    const int nvalid = m.cols - pcol < 8 ? m.cols - pcol : 8;
    if (m.param) {
        if (m.src_dtype == MUON_AMD_SRC_BF16) {
            uint16_t* const p = static_cast<uint16_t*>(m.param) + e;
            if (full) {
                const u32x4 pv = __builtin_nontemporal_load((const __attribute__((address_space(1))) u32x4*)(p));
                u32x4 r;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const float lo = round_bf(fmaf(ap.neg_lr, us[2 * k], round_bf(__uint_as_float(pv[k] << 16) * ap.wd_factor)));
                    const float hi = round_bf(fmaf(ap.neg_lr, us[2 * k + 1], round_bf(__uint_as_float(pv[k] & 0xffff0000u) * ap.wd_factor)));
                    r[k] = pack2bf(lo, hi);
                }
                __builtin_nontemporal_store(r, (__attribute__((address_space(1))) u32x4*)(p));
            } else {
                for (int k = 0; k < nvalid; ++k)
                    p[k] = f2bf(fmaf(ap.neg_lr, us[k], round_bf(bf2f(p[k]) * ap.wd_factor)));
            }
        } else {
            float* const p = static_cast<float*>(m.param) + e;
            if (full) {
                typedef float f32x4g __attribute__((ext_vector_type(4)));
                f32x4g p0 = __builtin_nontemporal_load((const __attribute__((address_space(1))) f32x4g*)(p));
                f32x4g p1 = __builtin_nontemporal_load((const __attribute__((address_space(1))) f32x4g*)(p + 4));
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    p0[k] = fmaf(ap.neg_lr, us[k], p0[k] * ap.wd_factor);
                    p1[k] = fmaf(ap.neg_lr, us[4 + k], p1[k] * ap.wd_factor);
                }
                __builtin_nontemporal_store(p0, (__attribute__((address_space(1))) f32x4g*)(p));
                __builtin_nontemporal_store(p1, (__attribute__((address_space(1))) f32x4g*)(p + 4));
            } else {
                for (int k = 0; k < nvalid; ++k) p[k] = fmaf(ap.neg_lr, us[k], p[k] * ap.wd_factor);
            }
        }
    }
    if (m.out) {
        uint16_t* const o = m.out + e;
        if (full) {
            u32x4 r;
#pragma unroll
            for (int k = 0; k < 4; ++k) r[k] = pack2bf(us[2 * k], us[2 * k + 1]);
            *(__attribute__((address_space(1))) u32x4*)(o) = r;
        } else {
            for (int k = 0; k < nvalid; ++k) o[k] = f2bf(us[k]);
        }
    }
}

// The addend: the lane that owns row (a*32 + lr) needs columns b*32 + 8q + 4g .. +4 of it.  Fetched
// that way from global memory, every load instruction would touch 32 different rows for 16 bytes
// each and the address pipe would take longer than the whole rest of the epilogue.  So the wave's
// WM x 64 piece of D is first streamed into its staging area `stage_d` (WM rows of 128 bytes) by
// the DMA path, one instruction per 8 full rows (chunks XOR-swizzled as in the operand ring), and
// the row-owning 8-byte pieces are read from LDS.  All of them are in registers when this returns:
// before any store of the sub-tile (D may alias C: in-place a*X + B*X).
template <int WGN, int WM, int WN, int TM, int TN>
__device__ __forceinline__ void ns_epilogue_addend(u32x2 (&dv)[TM][TN][4], const MuonGemmDesc& d,
                                                   const MuonTileJob& job, const char* stage_d) {
    static_assert(WN == 64, "the addend staging assumes 128-byte rows");
    int tid_e = threadIdx.x;
    asm volatile("" : "+v"(tid_e));            // see ns_epilogue_strips
    const int lane = tid_e & 63, wave = __builtin_amdgcn_readfirstlane(tid_e >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const int lr = lane & 31, g = lane >> 5;
    const int row0 = job.i0 + wm * WM, col0 = job.j0 + wn * WN;
    const uint32_t stage_lds = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(
        reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) char*)stage_d)));
    const int drow = lane >> 3;                         // row within the 8 rows of one instruction
    const u32x4 rsrc_d = dma_resource(d.D);
#pragma unroll
    for (int j = 0; j < WM / 8; ++j) {
        const int rr = j * 8 + drow;
        const int lc = (lane & 7) ^ ((rr >> 1) & 7);    // logical 16-byte chunk this lane fetches
        dma16(rsrc_d, static_cast<uint32_t>((static_cast<size_t>(row0 + rr) * d.ldd + col0 + lc * 8) * 2), 0u,
              stage_lds + j * 1024);
    }
    NS_WAIT_VMCNT(0);
#pragma unroll
    for (int a = 0; a < TM; ++a) {
        const int rr = a * 32 + lr;
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int q = 0; q < 4; ++q)
                dv[a][b][q] = *reinterpret_cast<const u32x2*>(
                    stage_d + rr * 128 + (((b * 4 + q) ^ ((rr >> 1) & 7)) * 16) + g * 8);
    }
}

// Wave-private staging bytes of the result strips: one 32-row strip in the direct orientation, then
// (in the same place) the strip's WN rows of 32 columns in the transposed one; rows padded by 16 B.
constexpr int strip_stage_bytes(int WN) {
    return 32 * (WN * 2 + 16) > WN * (32 * 2 + 16) ? 32 * (WN * 2 + 16) : WN * (32 * 2 + 16);
}

// Per 32-row strip of the wave's sub-tile, per 32 x 32 tile of it: t1 = alpha*acc -> row-owning
// layout -> + beta*D -> o (bf16) -> staged row-major in LDS -> 16-byte coalesced stores of C (and
// gamma*o to C2); o moved back to the column-owning layout -> staged -> 16-byte coalesced stores
// of CT (and C2T).  With APPLY, the orientation of the parameter goes through the fused parameter
// step instead of a store, and the other orientation is not produced.  `stage` is this wave's
// strip_stage_bytes(WN) of LDS.
// ROWSUM (a mirrored product without addend): per row of the result, the sum of |o| over the
// wave's 64 columns goes to d.rowsum[row][col0 / 64]; for a mirrored tile the column sums over the
// wave's WM rows go to the rows of the mirror image, d.rowsum[col][row0 / 64] (and zero to the other
// slots of those WM rows), so that every slot of every row is written exactly once per launch.
template <bool HAS_D, bool STREAM, bool APPLY, bool ROWSUM, int WGN, int WM, int WN, int TM, int TN>
__device__ __forceinline__ void ns_epilogue_strips(f32x16 (&acc)[TM][TN], const u32x2 (&dv)[TM][TN][4],
                                                   const MuonGemmDesc& d, const MuonTileJob& job, float alpha,
                                                   float beta, float gamma, bool round_terms, char* stage,
                                                   const ApplyArgs& ap) {
    constexpr int DROW = WN * 2 + 16;   // staged row pitch in bytes, direct orientation (32 rows)
    constexpr int TROW = 32 * 2 + 16;   // transposed orientation (WN rows of one strip's 32 columns)
    // The thread index goes through an opaque move here: everything the epilogue derives from it
    // is then computed after the main loop instead of being hoisted above it, where it would sit
    // in registers the loop needs (and be spilled to scratch memory by every wave).
    int tid_e = threadIdx.x;
    asm volatile("" : "+v"(tid_e));
    const int lane = tid_e & 63, wave = __builtin_amdgcn_readfirstlane(tid_e >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const int lr = lane & 31, g = lane >> 5;
    const int row0 = job.i0 + wm * WM, col0 = job.j0 + wn * WN;   // origin of this wave's sub-tile
    // X is the parameter itself for a wide parameter and its transpose for a tall one
    const bool apply_t = APPLY && ap.mat->rows > ap.mat->cols;
    const bool do_d = APPLY ? !apply_t : d.C != nullptr;
    const bool do_t = APPLY ? apply_t : (d.CT != nullptr && !(job.diag && d.CT == d.C));

    bf16x8 id0, id1;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const int rho = 8 * (t >> 2) + 4 * g + (t & 3);
        id0[t] = static_cast<__bf16>(rho == lr ? 1.0f : 0.0f);
        id1[t] = static_cast<__bf16>(16 + rho == lr ? 1.0f : 0.0f);
    }

    float colsum[TN];          // ROWSUM: |o| summed down this lane's 16 rows of every strip, per column tile
#pragma unroll
    for (int b = 0; b < TN; ++b) colsum[b] = 0.f;
#pragma unroll
    for (int a = 0; a < TM; ++a) {
        uint32_t ot[TN][8];   // this strip's results moved back to accumulator layout, packed bf16 pairs
        float rowpart = 0.f;  // ROWSUM: |o| summed along this lane's 32 of the strip's 64 columns
#pragma unroll
        for (int b = 0; b < TN; ++b) {
            if (round_terms) {
                // Every term rounded to bf16 as the reference's tensor expressions round.  Values
                // stay packed two bf16 per register from the conversion that rounds them: the pairs
                // are what the transposing MFMAs, the staging stores and the next conversion take.
                uint32_t p1[8];       // bf16(alpha * acc), accumulator layout
#pragma unroll
                for (int k = 0; k < 8; ++k) p1[k] = pack2bf(alpha * acc[a][b][2 * k], alpha * acc[a][b][2 * k + 1]);
                const f32x16 u = tile_transpose_packed(p1, id0, id1);
                uint32_t po[8];       // o = bf16(u + bf16(beta * D)), row-owning layout
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    if (HAS_D) {
                        const uint32_t t01 = pack2bf(beta * bf_lo(dv[a][b][q].x), beta * bf_hi(dv[a][b][q].x));
                        const uint32_t t23 = pack2bf(beta * bf_lo(dv[a][b][q].y), beta * bf_hi(dv[a][b][q].y));
                        po[2 * q] = pack2bf(u[4 * q] + bf_lo(t01), u[4 * q + 1] + bf_hi(t01));
                        po[2 * q + 1] = pack2bf(u[4 * q + 2] + bf_lo(t23), u[4 * q + 3] + bf_hi(t23));
                    } else {          // u holds bf16 values: exact
                        po[2 * q] = pack2bf(u[4 * q], u[4 * q + 1]);
                        po[2 * q + 1] = pack2bf(u[4 * q + 2], u[4 * q + 3]);
                    }
                    if constexpr (ROWSUM) {       // one term after the other, in column order
                        rowpart += fabsf(bf_lo(po[2 * q]));
                        rowpart += fabsf(bf_hi(po[2 * q]));
                        rowpart += fabsf(bf_lo(po[2 * q + 1]));
                        rowpart += fabsf(bf_hi(po[2 * q + 1]));
                    }
                    if (do_d)
                        *reinterpret_cast<u32x2*>(stage + lr * DROW + (b * 32 + 8 * q + 4 * g) * 2) =
                            u32x2{po[2 * q], po[2 * q + 1]};
                }
                if (do_t) {
                    if (HAS_D) {
                        const f32x16 w = tile_transpose_packed(po, id0, id1);
#pragma unroll
                        for (int k = 0; k < 8; ++k) ot[b][k] = pack2bf(w[2 * k], w[2 * k + 1]);
                    } else {
                        // without an addend o is the transposed t1, and its transpose is t1 again
#pragma unroll
                        for (int k = 0; k < 8; ++k) ot[b][k] = p1[k];
                        if constexpr (ROWSUM) {
#pragma unroll
                            for (int k = 0; k < 8; ++k) {
                                colsum[b] += fabsf(bf_lo(p1[k]));
                                colsum[b] += fabsf(bf_hi(p1[k]));
                            }
                        }
                    }
                }
                continue;
            }
            // One rounding per output: keep ~16 mantissa bits of alpha * acc through the transpose by
            // moving a bf16 head and a bf16 tail and adding them.
            f32x16 u;
            {
                float hi[16], lo[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float v = alpha * acc[a][b][i];
                    hi[i] = round_bf(v);
                    lo[i] = round_bf(v - hi[i]);
                }
                const f32x16 uh = tile_transpose_bf16(hi, id0, id1);
                const f32x16 ul = tile_transpose_bf16(lo, id0, id1);
#pragma unroll
                for (int i = 0; i < 16; ++i) u[i] = uh[i] + ul[i];
            }
            float o[16];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float dd[4] = {0.f, 0.f, 0.f, 0.f};
                if (HAS_D) {
                    dd[0] = bf_lo(dv[a][b][q].x);
                    dd[1] = bf_hi(dv[a][b][q].x);
                    dd[2] = bf_lo(dv[a][b][q].y);
                    dd[3] = bf_hi(dv[a][b][q].y);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    o[4 * q + e] = round_bf(u[4 * q + e] + (HAS_D ? beta * dd[e] : 0.f));
                    if constexpr (ROWSUM) rowpart += fabsf(o[4 * q + e]);
                }
                if (do_d) {
                    u32x2 pk;
                    pk.x = pack2bf(o[4 * q], o[4 * q + 1]);
                    pk.y = pack2bf(o[4 * q + 2], o[4 * q + 3]);
                    *reinterpret_cast<u32x2*>(stage + lr * DROW + (b * 32 + 8 * q + 4 * g) * 2) = pk;
                }
            }
            if (do_t) {
                const f32x16 w = tile_transpose_bf16(o, id0, id1);
#pragma unroll
                for (int k = 0; k < 8; ++k) ot[b][k] = pack2bf(w[2 * k], w[2 * k + 1]);
                if constexpr (ROWSUM) {
#pragma unroll
                    for (int k = 0; k < 16; ++k) colsum[b] += fabsf(w[k]);
                }
            }
        }
        if constexpr (ROWSUM) {
            // the partner lane (l ^ 32) owns the other 32 columns of the same row
            const float total = rowpart + __shfl_xor(rowpart, 32, 64);
            if (g == 0)
                d.rowsum[static_cast<size_t>(row0 + a * 32 + lr) * d.ld_rowsum + col0 / 64] = total;
        }
        if (do_d) {
            // 16-byte chunks per row, whole rows per wave-wide store
            constexpr int CPR = WN / 8, RPI = 64 / CPR;
            const int r = lane / CPR, ch = lane % CPR;
            if constexpr (APPLY) {
#pragma unroll 1
                for (int it = 0; it < 32 / RPI; ++it) {
                    const int row = it * RPI + r;
                    const u32x4 v = *reinterpret_cast<const u32x4*>(stage + row * DROW + ch * 16);
                    apply_chunk8(ap, row0 + a * 32 + row, col0 + ch * 8, v);
                }
            } else {
#pragma unroll
                for (int it = 0; it < 32 / RPI; ++it) {
                    const int row = it * RPI + r;
                    const u32x4 v = *reinterpret_cast<const u32x4*>(stage + row * DROW + ch * 16);
                    const size_t off = static_cast<size_t>(row0 + a * 32 + row) * d.ldc + col0 + ch * 8;
                    gstore16<STREAM>(d.C + off, v);
                    if (d.C2) gstore16<STREAM>(d.C2 + off, scale_bf16x8(v, gamma));
                }
            }
        }
        if (do_t) {
#pragma unroll
            for (int b = 0; b < TN; ++b)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    u32x2 pk;
                    pk.x = ot[b][2 * q];
                    pk.y = ot[b][2 * q + 1];
                    *reinterpret_cast<u32x2*>(stage + (b * 32 + lr) * TROW + (8 * q + 4 * g) * 2) = pk;
                }
            constexpr int CPR = 32 / 8, RPI = 64 / CPR;
            const int r = lane / CPR, ch = lane % CPR;
            if constexpr (APPLY) {
#pragma unroll 1
                for (int it = 0; it < WN / RPI; ++it) {
                    const int row = it * RPI + r;
                    const u32x4 v = *reinterpret_cast<const u32x4*>(stage + row * TROW + ch * 16);
                    apply_chunk8(ap, col0 + row, row0 + a * 32 + ch * 8, v);
                }
            } else {
#pragma unroll
                for (int it = 0; it < WN / RPI; ++it) {
                    const int row = it * RPI + r;
                    const u32x4 v = *reinterpret_cast<const u32x4*>(stage + row * TROW + ch * 16);
                    const size_t off = static_cast<size_t>(col0 + row) * d.ldct + row0 + a * 32 + ch * 8;
                    gstore16<STREAM>(d.CT + off, v);
                    if (d.C2T) gstore16<STREAM>(d.C2T + off, scale_bf16x8(v, gamma));
                }
            }
        }
    }
    if constexpr (ROWSUM) {
        if (do_t) {
#pragma unroll
            for (int b = 0; b < TN; ++b) {
                // the partner lane owns the other 16 rows of every strip of the same column
                const float total = colsum[b] + __shfl_xor(colsum[b], 32, 64);
                if (g == 0) {
                    float* const dst = d.rowsum + static_cast<size_t>(col0 + b * 32 + lr) * d.ld_rowsum + row0 / 64;
                    dst[0] = total;
#pragma unroll
                    for (int z = 1; z < WM / 64; ++z) dst[z] = 0.f;
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// The kernel
// ---------------------------------------------------------------------------------------------
// The LDS ring holds NHALF half-stages; a half-stage is the P rows or the Q rows of one k-block
// (BT rows x 128 bytes).  Half-stages are issued in the order P0 Q0 P1 Q1 P2 ...; block kb needs
// halves 2kb and 2kb+1.  The prologue issues the first NHALF; the pair 2kb+NHALF, 2kb+NHALF+1 goes
// into the two slots of block kb, from the last k-step of block kb (every fragment of the block is
// in registers by then) through the first three k-steps of block kb+1.  So while a block is
// multiplied the next one and a half are in flight or landed, the load pipe always has queued
// requests, and every request is a full 128-byte line.  NHALF = 5 fills the 160 KB LDS for the
// 256 x 256 tile.
#ifndef NS_SPLIT_TICKET_ORDER
#define NS_SPLIT_TICKET_ORDER __ATOMIC_RELEASE
#endif

template <int BT_, int WGM_, int WGN_, int MINB_, int NHALF_, bool SPLIT_K_>
struct GemmCfg {
    static constexpr bool SPLIT_K = SPLIT_K_;     // jobs may share a tile's reduction
    static constexpr bool STREAM_STORES = BT_ >= 256;   // see gstore16
    // A second copy of the k-block without the tests of the first and last blocks (see NS_KBLOCK).
    // The 256 x 256 class has no registers to spare for the moves between two copies of its loop.
    static constexpr bool STEADY_LOOP = BT_ < 256;
    static constexpr int BM = BT_, BN = BT_, WGM = WGM_, WGN = WGN_, MINB = MINB_, NHALF = NHALF_;
    static constexpr int NW = WGM * WGN, NT = NW * 64;
    static constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
    static constexpr int HALF_BYTES = BT_ * ROW_BYTES;
    static constexpr int DPH = BT_ / 8 / NW;          // DMA instructions (8 rows each) per wave per half
    static constexpr size_t RING_BYTES = static_cast<size_t>(NHALF) * HALF_BYTES;
    static constexpr size_t LDS_BYTES = RING_BYTES;
    // After the main loop the ring is free.  The addend pieces (WM rows of 128 bytes per wave) are
    // staged at its start; once they are in registers, the first NPRE half-stages of the
    // workgroup's next job are fetched into slots 0 .. NPRE-1 while the result strips are staged
    // behind them.
    static constexpr int NPRE = 3;
    static constexpr size_t ADDEND_BYTES = static_cast<size_t>(NW) * WM * 128;
    static constexpr size_t STRIP_OFFSET = static_cast<size_t>(NPRE) * HALF_BYTES;
    static constexpr size_t STRIP_BYTES = strip_stage_bytes(WN);
    static_assert(ADDEND_BYTES <= RING_BYTES, "addend staging");
    static_assert(STRIP_OFFSET + NW * STRIP_BYTES <= RING_BYTES, "strip staging behind the prefetched halves");
    static_assert(BT_ % (8 * NW) == 0, "DMA tiling");
    static_assert((NHALF - 2) * DPH < 64 && NHALF >= 5, "vmcnt immediate / ring depth");
    static_assert(NW % 2 == 0, "swizzle parity assumes an even wave count");
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be MFMA tiles");
    static_assert(LDS_BYTES <= 163840, "LDS capacity of a gfx950 CU");
};

// A launch is persistent: it has as many workgroups as the GPU holds at once (or one per job when
// there are fewer jobs), and workgroup b computes jobs b, b + gridDim.x, b + 2 gridDim.x, ... of the
// list.  Workgroups are dealt round-robin to the XCDs, so with a grid that is a multiple of 8 job j
// still runs on XCD j % 8, in list order.  Between two jobs of a workgroup nothing waits for a
// launch: the descriptors of the next job are read while the addend of the current one is in
// flight, and its first NPRE half-stages stream into LDS while the epilogue of the current one
// runs.
// APPLY: the launch is the last update product of the iteration and its epilogue takes the
// parameter step (mats[job.desc] describes the parameter of the job's matrix; `sc`, when given,
// holds {lr, wd_factor} in device memory and overrides the by-value arguments).
// QK: the second operand is given k-major, Q[k][j] with leading dimension ldq (acc[i][j] = sum_k
// P[i][k] Q[k][j]: the update a X + B X reads X itself, no transposed copy of it exists); its
// half-stage is then BK rows of BN columns, fetched in the same 1 KiB pieces.
template <typename Cfg, bool APPLY, bool QK>
__global__ __launch_bounds__(Cfg::NT, Cfg::MINB) void ns_gemm_kernel(
    const MuonGemmDesc* __restrict__ descs, const MuonTileJob* __restrict__ jobs, int njobs, float alpha,
    float beta, float gamma, int flags, float* __restrict__ split_partials,
    int32_t* __restrict__ split_counters, const MuonMatDesc* __restrict__ mats, float neg_lr,
    float wd_factor, const float* __restrict__ sc) {
    constexpr int NW = Cfg::NW, WGN = Cfg::WGN, WM = Cfg::WM, WN = Cfg::WN;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, HALF_BYTES = Cfg::HALF_BYTES, DPH = Cfg::DPH;
    constexpr int NHALF = Cfg::NHALF, NPRE = Cfg::NPRE;
    constexpr int ROWQ = Cfg::BN * 2;           // bytes of one k-row of a k-major Q half-stage
    static_assert(!APPLY || QK, "the parameter step rides the update product, whose second operand is k-major");
    extern __shared__ __align__(16) uint16_t lds[];
    const int tid = threadIdx.x;
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
        (__attribute__((address_space(3))) uint16_t*)lds));

    // ---- DMA addressing: instruction j of this wave fills half-stage rows (j*NW + wave)*8 .. +8;
    //      lane -> row + lane/8, LDS chunk position lane%8, i.e. global chunk (lane%8) ^ swizzle,
    //      swizzle = (row >> 1) & 7 = 4*(wave & 1) + lane/16 ---------------------------------------
    // The per-lane constants of the main loop are derived once per job from an opaque copy of the
    // thread index: they are a few instructions, and kept across the epilogue they would cost it
    // registers it does not have.
#define NS_LANE_CONSTANTS()                                                                    \
    int tid_l = tid;                                                                           \
    asm volatile("" : "+v"(tid_l));                                                            \
    const int lane = tid_l & 63, wave = __builtin_amdgcn_readfirstlane(tid_l >> 6);            \
    const int wm = wave / WGN, wn = wave % WGN;                                                \
    const int gchunk = (lane & 7) ^ (((wave & 1) << 2) | (lane >> 4));                         \
    const uint32_t dst0 = lds_base + wave * 1024
    // k-major Q: piece (j*NW + wave) of the half-stage is 1024 / ROWQ whole k-rows; lane -> k-row
    // and 16-byte position in it; the 64-byte block at position pb of row k holds the row's block
    // pb ^ (k & 3) (the transposing fragment reads of four consecutive k then hit different banks).
    uint32_t srcp[DPH];                         // per-lane byte offsets of this wave's pieces in P and Q
    uint32_t srcq[DPH];
    u32x4 rsrc_p, rsrc_q;                       // (wave-uniform: they live in scalar registers)
    uint32_t qstep;                             // bytes from one k-block of Q to the next
#define NS_SET_SOURCES(job_, d_)                                                               \
    do {                                                                                       \
        _Pragma("unroll") for (int j_ = 0; j_ < DPH; ++j_) {                                   \
            const int r_ = (j_ * NW + wave) * 8 + (lane >> 3);                                 \
            srcp[j_] = static_cast<uint32_t>((static_cast<size_t>((job_).i0 + r_) * (d_).ldp + (job_).k0 + gchunk * 8) * 2); \
            if constexpr (QK) {                                                                \
                const int o_ = (j_ * NW + wave) * 1024 + lane * 16;                            \
                const int k_ = o_ / ROWQ, w_ = o_ % ROWQ;                                      \
                const int col_ = (((w_ >> 6) ^ (k_ & 3)) << 5) + ((w_ & 63) >> 1);             \
                srcq[j_] = static_cast<uint32_t>((static_cast<size_t>((job_).k0 + k_) * (d_).ldq + (job_).j0 + col_) * 2); \
            } else {                                                                           \
                srcq[j_] = static_cast<uint32_t>((static_cast<size_t>((job_).j0 + r_) * (d_).ldq + (job_).k0 + gchunk * 8) * 2); \
            }                                                                                  \
        }                                                                                      \
        rsrc_p = dma_resource((d_).P);                                                         \
        rsrc_q = dma_resource((d_).Q);                                                         \
        qstep = QK ? static_cast<uint32_t>(BK * 2) * (d_).ldq : static_cast<uint32_t>(BK * 2); \
    } while (0)

    // half h = 2*kb (+1): P (Q) rows of k-block kb, into ring slot h % NHALF
#define NS_ISSUE_HALF(rsrc_, src_, step_, kb_, slot_)                                          \
    do {                                                                                       \
        _Pragma("unroll") for (int j_ = 0; j_ < DPH; ++j_)                                     \
            dma16(rsrc_, src_[j_], static_cast<uint32_t>(kb_) * (step_),                       \
                  dst0 + (slot_) * HALF_BYTES + j_ * NW * 1024);                               \
    } while (0)
    // the first halves of a job, h in [H0_, H1_) and below 2*nk_: P0 Q0 P1 Q1 P2 ... into slots 0 1 2 ...
#define NS_ISSUE_FIRST_HALVES(H0_, H1_, nk_)                                                   \
    do {                                                                                       \
        _Pragma("unroll") for (int h_ = (H0_); h_ < (H1_); ++h_) {                             \
            if (h_ < 2 * (nk_)) {                                                              \
                if (h_ & 1) NS_ISSUE_HALF(rsrc_q, srcq, qstep, h_ >> 1, h_);                   \
                else NS_ISSUE_HALF(rsrc_p, srcp, static_cast<uint32_t>(BK * 2), h_ >> 1, h_);  \
            }                                                                                  \
        }                                                                                      \
    } while (0)

    constexpr int KSTEPS = BK / 16;
    constexpr int DPK = 2 * DPH / KSTEPS;                    // DMA instructions per k-step
    static_assert(2 * DPH % KSTEPS == 0 && DPH % DPK == 0, "DMA instructions must spread evenly");
    static_assert(KSTEPS % 2 == 0, "the fragments read at a block's last k-step land in buffer 0");
    static_assert(DPK <= TM, "one DMA instruction per row of MFMAs");

    const bool round_terms = (flags & MUON_AMD_ROUND_REFERENCE) != 0;
    if constexpr (APPLY) {
        if (sc) {
            neg_lr = -sc[0];
            wd_factor = sc[1];
        }
    }

    int job_idx = blockIdx.x;                   // the launcher never starts more workgroups than jobs
    MuonTileJob job = jobs[job_idx];
    MuonGemmDesc d = descs[job.desc];
    int nk = (job.k1 - job.k0) / BK;            // this job's share of the reduction
    {
        NS_LANE_CONSTANTS();
        (void)wm;
        (void)wn;
        NS_SET_SOURCES(job, d);
        NS_ISSUE_FIRST_HALVES(0, NHALF, nk);    // prologue: halves 0 .. NHALF-1
    }

    for (;;) {
        NS_LANE_CONSTANTS();
        // ---- fragment addressing (bytes): lane l reads row l%32, chunk 2*ks + l/32 -------------
        const int swz = (lane >> 1) & 7;
        const int c0 = (lane >> 5) ^ swz;
        const uint32_t pfrag_off = (wm * WM + (lane & 31)) * ROW_BYTES;
        const uint32_t qfrag_off = (wn * WN + (lane & 31)) * ROW_BYTES;
        // k-major Q: lane l addresses row 8 (l / 32) + (l % 16) / 4 of the k-step, columns
        // 32 b + 16 ((l / 16) % 2) + 4 (l % 4) .. + 3 of the wave's 64, in the swizzled block
        uint32_t qtr_off[TN];
        if constexpr (QK) {
            const int r4 = (lane & 15) >> 2;
#pragma unroll
            for (int b = 0; b < TN; ++b)
                qtr_off[b] = ((lane >> 5) * 8 + r4) * ROWQ + (((wn * (WN / 32) + b) ^ r4) << 6) +
                             ((lane >> 4) & 1) * 32 + (lane & 3) * 8;
        }
        const int koff[4] = {c0 * 16, (c0 ^ 2) * 16, (c0 ^ 4) * 16, (c0 ^ 6) * 16};
        // the sources of the halves beyond the first ones (set again: the copies made when the
        // first halves were issued are not kept across the epilogue before)
        NS_SET_SOURCES(job, d);

        f32x16 acc[TM][TN];
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int b = 0; b < TN; ++b)
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;

        // Block 0 has landed once only the younger first halves are pending (for a job after the
        // first, halves 0 .. NPRE-1 landed long ago and at most NHALF - NPRE are pending).
        WaitHalves<DPH, NHALF - 2>::run((2 * nk < NHALF ? 2 * nk : NHALF) - 2);
        __syncthreads();

        // Fragments are double buffered over k-steps ACROSS blocks: the ds_reads of the next k-step
        // (the first one of block kb+1 included) are issued ahead of the MFMAs of the current one, so
        // the matrix pipe never waits for LDS latency, not even right after the barrier.  The reads
        // and the waits for them are written out (FragLoad, wait_frags): LDS reads return in order,
        // so "at most TM + TN outstanding" means the fragments of the current k-step have arrived
        // while those just requested are still in flight.  Left to the compiler, the wait at the
        // join after the last block's branch covered the reads issued right after the barrier.
        // The compiler takes a register written by FragLoad as valid at once: between a read and
        // its wait there must be no place where it may copy that register (no loop edge, no join
        // of paths that define it differently).
        u32x4 af[2][TM], bfr[2][TN];
        u32x2 btr[2][2 * TN];               // k-major Q: the halves (k 0..3, k 4..7 of a lane) of its fragments
        constexpr int NFRAG = TM + (QK ? 2 * TN : TN);      // LDS reads of one k-step
        const uint32_t pfrag_a = lds_base + pfrag_off;
        const uint32_t qfrag_a = lds_base + qfrag_off;
#define NS_LOAD_FRAGS(buf_, sp_, sq_, ks_)                                                      \
    do {                                                                                       \
        FragLoad<TM>::run(af[buf_], pfrag_a + (sp_) * HALF_BYTES + koff[ks_]);                 \
        if constexpr (QK)                                                                      \
            FragLoadTr<TN, ROWQ>::run(btr[buf_], qtr_off, lds_base + (sq_) * HALF_BYTES + (ks_) * 16 * ROWQ); \
        else                                                                                   \
            FragLoad<TN>::run(bfr[buf_], qfrag_a + (sq_) * HALF_BYTES + koff[ks_]);            \
    } while (0)
#define NS_WAIT_FRAGS(CNT_, buf_)                                                               \
    do {                                                                                       \
        if constexpr (QK) wait_frags_tr<CNT_>(af[buf_], btr[buf_]);                            \
        else wait_frags<CNT_>(af[buf_], bfr[buf_]);                                            \
    } while (0)
        NS_LOAD_FRAGS(0, 0, 1, 0);
        NS_WAIT_FRAGS(0, 0);               // (once per tile) nothing in flight on entry to the loop either

        // The pair of halves being issued: created at the barrier of block kb (last k-step), its
        // 2*DPH DMA instructions are spread over that k-step and the first KSTEPS-1 of block kb+1,
        // one after each of the first DPK rows of MFMAs -- a burst right after the barrier would hold
        // every wave in the memory-issue queue while the matrix pipe sits idle.
        // NHALF odd: the first half of a pair is a Q half (needed one block earlier), the second P.
        const uint32_t* const dsrc[2] = {(NHALF & 1) ? srcq : srcp, (NHALF & 1) ? srcp : srcq};
        const u32x4 drsrc[2] = {(NHALF & 1) ? rsrc_q : rsrc_p, (NHALF & 1) ? rsrc_p : rsrc_q};
        uint32_t ddst[2] = {0, 0};
        uint32_t dk[2] = {0, 0};           // byte offset of the k-block being fetched, per half of the pair
        const uint32_t dstep[2] = {(NHALF & 1) ? qstep : static_cast<uint32_t>(BK * 2), (NHALF & 1) ? static_cast<uint32_t>(BK * 2) : qstep};
        bool dgo[2] = {false, false};

        // One k-block.  STEADY_: a block in the middle of a long reduction -- both halves of the pair
        // created at the previous barrier and the first half of the pair created at this one exist
        // (1 <= kb <= nk - 3), so every DMA instruction is issued without a test and the wait before
        // the barrier is a constant; the first block and the last two take the general form.
#define NS_KBLOCK(STEADY_)                                                                      \
    do {                                                                                       \
        int spn = sp + 2; spn = spn >= NHALF ? spn - NHALF : spn;                              \
        int sqn = sq + 2; sqn = sqn >= NHALF ? sqn - NHALF : sqn;                              \
        _Pragma("unroll") for (int ks = 0; ks < KSTEPS; ++ks) {                                \
            const int cur = ks & 1, nxt = cur ^ 1;                                             \
            if (ks + 1 < KSTEPS) {                                                             \
                NS_LOAD_FRAGS(nxt, sp, sq, ks + 1);                                            \
                NS_WAIT_FRAGS(NFRAG, cur);                                                     \
            } else {                                                                           \
                /* Every fragment of block kb is in registers.  Block kb+1 has landed once only   \
                   the younger halves are pending; after the barrier it is visible to all waves   \
                   and the two slots of block kb are free for the next pair of halves,            \
                   2kb+NHALF and 2kb+NHALF+1. */                                                  \
                NS_WAIT_FRAGS(0, cur);                                                         \
                if (STEADY_ || kb + 1 < nk) {                                                  \
                    if (STEADY_) {                                                             \
                        NS_WAIT_VMCNT((NHALF - 4) * DPH);                                      \
                    } else {                                                                   \
                        const int issued = 2 * nk < 2 * kb + NHALF ? 2 * nk : 2 * kb + NHALF;  \
                        WaitHalves<DPH, NHALF - 2>::run(issued - (2 * kb + 4));                \
                    }                                                                          \
                    __builtin_amdgcn_s_barrier();                                              \
                    const int h0 = 2 * kb + NHALF;                                             \
                    ddst[0] = dst0 + sp * HALF_BYTES;            /* h0 % NHALF == 2kb % NHALF */  \
                    ddst[1] = dst0 + sq * HALF_BYTES;                                          \
                    dk[0] = static_cast<uint32_t>(h0 >> 1) * dstep[0];                         \
                    dk[1] = static_cast<uint32_t>((h0 + 1) >> 1) * dstep[1];                   \
                    dgo[0] = h0 < 2 * nk;                                                      \
                    dgo[1] = h0 + 1 < 2 * nk;                                                  \
                } else {                                                                       \
                    dgo[0] = dgo[1] = false;     /* last block: nothing left to fetch */       \
                }                                                                              \
                /* The first fragments of block kb+1, read under the last MFMAs of block kb.      \
                   After the last block the same reads go out and their result is not used: the   \
                   fragment registers then have one definition on every path, so the compiler has \
                   no reason to copy them while the reads are in flight. */                       \
                NS_LOAD_FRAGS(nxt, spn, sqn, 0);                                               \
            }                                                                                  \
            __builtin_amdgcn_sched_barrier(0);   /* keep these reads ahead of the MFMAs below */  \
            _Pragma("unroll") for (int a = 0; a < TM; ++a) {                                   \
                _Pragma("unroll") for (int b = 0; b < TN; ++b) {                               \
                    u32x4 qv;                                                                  \
                    if constexpr (QK) qv = u32x4{btr[cur][2 * b].x, btr[cur][2 * b].y, btr[cur][2 * b + 1].x, btr[cur][2 * b + 1].y}; \
                    else qv = bfr[cur][b];                                                     \
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(                       \
                        __builtin_bit_cast(bf16x8, af[cur][a]), __builtin_bit_cast(bf16x8, qv), acc[a][b], 0, 0, 0); \
                }                                                                              \
                if (a < DPK) {                                                                 \
                    /* instruction jj of the current pair: the last k-step starts a pair */    \
                    const int jj = (ks + 1 < KSTEPS ? (ks + 1) * DPK : 0) + a;                 \
                    const int h = jj / DPH, j = jj % DPH;                                      \
                    __builtin_amdgcn_sched_barrier(0);                                         \
                    if (STEADY_ || dgo[h]) dma16(drsrc[h], dsrc[h][j], dk[h], ddst[h] + j * NW * 1024); \
                    __builtin_amdgcn_sched_barrier(0);                                         \
                }                                                                              \
            }                                                                                  \
            __builtin_amdgcn_sched_barrier(0);                                                 \
        }                                                                                      \
        /* Nothing is in flight across the end of a k-block: the reads issued before the last     \
           row of MFMAs have long arrived, and waiting for them here keeps every pending          \
           fragment inside one copy of this code (a register the compiler moved at a loop edge    \
           or between the two copies would be moved before its data is there). */                 \
        NS_WAIT_FRAGS(0, 0);                                                                   \
        sp = spn;                                                                              \
        sq = sqn;                                                                              \
    } while (0)

        int sp = 0, sq = 1;                 // ring slots of the P and Q halves of block kb
        for (int kb = 0; kb < nk;) {
            if constexpr (Cfg::STEADY_LOOP) {
                if (kb >= 1 && kb <= nk - 3) {
                    do {
                        NS_KBLOCK(true);
                        ++kb;
                    } while (kb <= nk - 3);
                    continue;
                }
            }
            NS_KBLOCK(false);
            ++kb;
        }
#undef NS_KBLOCK
#undef NS_WAIT_FRAGS
#undef NS_LOAD_FRAGS
        __syncthreads();            // every wave is done reading the ring: LDS becomes staging space

        const int next_idx = job_idx + static_cast<int>(gridDim.x);
        const bool has_next = next_idx < njobs;

        // ---- split reduction (small tile class only): a tile whose K range is shared by `count`
        //      jobs.  Each job parks its fp32 accumulators in its own slot; the job that arrives last
        //      adds the slots in slot order (so the sum does not depend on which job that is) and
        //      writes the tile.  Nobody waits for anybody: the other jobs go on to their next job.
        //      Hand-over: the slots are written with device-scope stores, which go through to memory
        //      past the XCD-private L2; after the workgroup barrier one thread takes the ticket with
        //      release order at device scope, so every slot store of the workgroup happens before
        //      the ticket is visible.  Only the one job per tile that adds the slots up pays for an
        //      acquire fence (which drops what its XCD's L2 holds of them) before its plain loads. ----
        bool write_tile = true;
        if constexpr (Cfg::SPLIT_K) {
            const int split_count = job.split >> 16;
            if (split_count > 1) {
                constexpr size_t TILE_ELEMS = static_cast<size_t>(Cfg::BM) * Cfg::BN;
                float* const mine = split_partials + (static_cast<size_t>(job.part_base) + (job.split & 0xffff)) * TILE_ELEMS;
                // (opaque, so that the 64 slot addresses derived from it are not hoisted out of the
                // job loop and carried in registers through the main loop)
                int tid_s = tid;
                asm volatile("" : "+v"(tid_s));
                const size_t lane_off = static_cast<size_t>(tid_s >> 6) * TM * TN * 16 * 64 + (tid_s & 63);
#pragma unroll
                for (int a = 0; a < TM; ++a)
#pragma unroll
                    for (int b = 0; b < TN; ++b)
#pragma unroll
                        for (int i = 0; i < 16; ++i)
                            __hip_atomic_store(&mine[lane_off + ((a * TN + b) * 16 + i) * 64], acc[a][b][i],
                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __builtin_amdgcn_s_waitcnt(0);                     // this wave's slot stores are acknowledged ...
                __syncthreads();
                int* const ticket = reinterpret_cast<int*>(lds);
                if (tid == 0)                                      // ... and the whole slot is out before I am counted
                    *ticket = __hip_atomic_fetch_add(&split_counters[job.part_base], 1, NS_SPLIT_TICKET_ORDER,
                                                     __HIP_MEMORY_SCOPE_AGENT);
                __syncthreads();
                const bool last = *ticket == split_count - 1;
                __syncthreads();                                   // the ticket is read before LDS is reused
                write_tile = last;
                if (last) {
                    if (tid == 0)                                  // ready for the next launch on the stream
                        __hip_atomic_store(&split_counters[job.part_base], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent"); // drop what this XCD cached of the slots
                    const float* const first = split_partials + static_cast<size_t>(job.part_base) * TILE_ELEMS;
#pragma unroll
                    for (int a = 0; a < TM; ++a)
#pragma unroll
                        for (int b = 0; b < TN; ++b)
#pragma unroll
                            for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;
                    // slot by slot, all of a lane's loads of one slot in flight together
                    for (int sidx = 0; sidx < split_count; ++sidx) {
                        const float* const slot = first + sidx * TILE_ELEMS;
#pragma unroll
                        for (int a = 0; a < TM; ++a) {
                            float t[TN][16];
#pragma unroll
                            for (int b = 0; b < TN; ++b)
#pragma unroll
                                for (int i = 0; i < 16; ++i) t[b][i] = slot[lane_off + ((a * TN + b) * 16 + i) * 64];
                            __builtin_amdgcn_sched_barrier(0);     // all of these loads go out before the first add waits
#pragma unroll
                            for (int b = 0; b < TN; ++b)
#pragma unroll
                                for (int i = 0; i < 16; ++i) acc[a][b][i] += t[b][i];
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
            }
        }

        // ---- epilogue, first part: the addend into registers (staged at the start of the ring) ----
        const bool has_d = APPLY || d.D != nullptr;
        u32x2 dv[TM][TN][4];
        if (write_tile && has_d) {
            ns_epilogue_addend<WGN, WM, WN, TM, TN>(dv, d, job, reinterpret_cast<const char*>(lds) + wave * (WM * 128));
        } else {
            // defined on every path, so that nothing of it is carried around the job loop in registers
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int b = 0; b < TN; ++b)
#pragma unroll
                    for (int q = 0; q < 4; ++q) dv[a][b][q] = u32x2{0u, 0u};
        }

        // ---- the next job's first half-stages stream in while the result strips are written -----
        // every wave holds its addend: the start of the ring is free for the next job's halves, and
        // the part of it under the strip staging of other waves may be overwritten
        if (write_tile && has_d) __syncthreads();

        // ---- the workgroup's next job: its first half-stages stream in while the result strips
        //      are written (its descriptors are read again after the strips rather than kept in
        //      registers across them) ------------------------------------------------------------
        if (has_next) {
            const MuonTileJob nj = jobs[next_idx];
            const MuonGemmDesc nd = descs[nj.desc];
            const int nnk = (nj.k1 - nj.k0) / BK;
            NS_SET_SOURCES(nj, nd);
            NS_ISSUE_FIRST_HALVES(0, NPRE, nnk);
        }
        const int wave_e = wave;      // (scalar) for the staging offsets below

        // ---- epilogue, second part: the result strips (staged behind the prefetched halves) ---------
        if (write_tile) {
            char* const stage = reinterpret_cast<char*>(lds) + Cfg::STRIP_OFFSET + wave_e * Cfg::STRIP_BYTES;
            ApplyArgs ap{nullptr, 0.f, 1.f, false};
            if constexpr (APPLY) {
                ap.mat = mats + job.desc;
                ap.neg_lr = neg_lr;
                ap.wd_factor = wd_factor;
                ap.vec_ok = (ap.mat->cols % 8 == 0) && ((reinterpret_cast<uintptr_t>(ap.mat->param) & 15) == 0) &&
                            ((reinterpret_cast<uintptr_t>(ap.mat->out) & 15) == 0);
                ns_epilogue_strips<true, Cfg::STREAM_STORES, true, false, WGN, WM, WN, TM, TN>(acc, dv, d, job, alpha, beta, gamma, round_terms, stage, ap);
            } else {
                if (has_d) ns_epilogue_strips<true, Cfg::STREAM_STORES, false, false, WGN, WM, WN, TM, TN>(acc, dv, d, job, alpha, beta, gamma, round_terms, stage, ap);
                else if ((flags & MUON_AMD_GEMM_ROWSUM) && d.rowsum) ns_epilogue_strips<false, Cfg::STREAM_STORES, false, true, WGN, WM, WN, TM, TN>(acc, dv, d, job, alpha, beta, gamma, round_terms, stage, ap);
                else ns_epilogue_strips<false, Cfg::STREAM_STORES, false, false, WGN, WM, WN, TM, TN>(acc, dv, d, job, alpha, beta, gamma, round_terms, stage, ap);
            }
        }
        if (!has_next) break;

        // The next job becomes the current one.  The index goes through an opaque move so that the
        // descriptors are loaded afresh (from the scalar cache) instead of living in registers
        // through the epilogue above.
        int idx = next_idx;
        asm volatile("" : "+s"(idx));
        job = jobs[idx];
        d = descs[job.desc];
        nk = (job.k1 - job.k0) / BK;
        {
            int tid_n = tid;
            asm volatile("" : "+v"(tid_n));
            const int lane = tid_n & 63, wave = __builtin_amdgcn_readfirstlane(tid_n >> 6);
            const int gchunk = (lane & 7) ^ (((wave & 1) << 2) | (lane >> 4));
            const uint32_t dst0 = lds_base + wave * 1024;
            NS_SET_SOURCES(job, d);
        // The strips of every wave are out of LDS (the stores that read them have been issued from
        // registers) and, with vmcnt at zero, the prefetched halves have landed: the rest of the
        // ring can take the remaining first halves, and the wait at the top of the loop sees only those.
            NS_WAIT_VMCNT(0);
            __syncthreads();
            NS_ISSUE_FIRST_HALVES(NPRE, NHALF, nk);
        }
        job_idx = idx;
    }
#undef NS_ISSUE_FIRST_HALVES
#undef NS_ISSUE_HALF
#undef NS_SET_SOURCES
#undef NS_LANE_CONSTANTS
}

// Tile classes: square output tile, waves, workgroups per CU.
//   0: 128 x 128, 4 waves of 64 x 64, two workgroups per CU   (short side below 1024)
//   1: 256 x 256, 8 waves of 128 x 64, one workgroup per CU   (large matrices)
#ifndef NS_CFG0_MINB
#define NS_CFG0_MINB 2
#define NS_CFG0_NHALF 5
#endif
typedef GemmCfg<128, 2, 2, NS_CFG0_MINB, NS_CFG0_NHALF, true> Cfg0;
typedef GemmCfg<256, 2, 4, 1, 5, false> Cfg1;
constexpr int kNumTileClasses = 2;

struct TileClass {
    int bm, bn, threads;
    size_t lds_bytes;
    bool split_k;
};
static const TileClass kTileClasses[kNumTileClasses] = {
    {Cfg0::BM, Cfg0::BN, Cfg0::NT, Cfg0::LDS_BYTES, Cfg0::SPLIT_K},
    {Cfg1::BM, Cfg1::BN, Cfg1::NT, Cfg1::LDS_BYTES, Cfg1::SPLIT_K},
};

// ---------------------------------------------------------------------------------------------
// Per-device set-up, done once per device with that device current: the device must be a gfx950,
// the kernels use more dynamic LDS than the default limit (raising it is not a stream operation,
// so it must not wait for the first launch, which may be one that a caller records into a HIP
// graph), and the address of this device's copy of the static scratch array is looked up.
// ---------------------------------------------------------------------------------------------
// Split-reduction scratch for callers that cannot allocate (muon_amd_ns_gemm_noalloc): the fp32
// slots of the 128 x 128 tile class followed by one int32 counter per slot.  Every GPU the
// library runs on holds its own copy until the process ends.  In host code the name `scratch`
// is only a handle for hipGetSymbolAddress; kernels are given the looked-up address.
constexpr int kStaticSplitSlots = MUON_AMD_NOALLOC_MAX_SPLIT_SLOTS;
constexpr size_t kStaticSlotBytes = static_cast<size_t>(Cfg0::BM) * Cfg0::BN * sizeof(float);
constexpr size_t kStaticCounterOffset = kStaticSplitSlots * kStaticSlotBytes;
constexpr size_t kStaticScratchBytes = kStaticCounterOffset + kStaticSplitSlots * sizeof(int32_t);
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
struct DeviceState {
    std::atomic<bool> ready{false};           // set (release) once the fields below are final
    int num_cus = 0;                          // a persistent launch has num_cus * MINB workgroups at most
    unsigned char* scratch_ptr = nullptr;     // device address of `scratch` on this device
};
static DeviceState g_devices[kMaxDevices];
static std::mutex g_devices_mutex;

template <typename Cfg, bool APPLY, bool QK>
static int raise_lds_limit() {
    auto kern = ns_gemm_kernel<Cfg, APPLY, QK>;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(Cfg::LDS_BYTES)) != hipSuccess) {
        (void)hipGetLastError();
        set_error("ns_gemm: cannot raise dynamic LDS to %zu bytes", Cfg::LDS_BYTES);
        return MUON_AMD_ELAUNCH;
    }
    return MUON_AMD_OK;
}

static int device_setup(const DeviceState** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        set_error("no usable HIP device is current (device index %d)", dev);
        return MUON_AMD_EDEVICE;
    }
    DeviceState& st = g_devices[dev];
    if (st.ready.load(std::memory_order_acquire)) {     // every launch after the first: no lock
        *out = &st;
        return MUON_AMD_OK;
    }
    std::lock_guard<std::mutex> lock(g_devices_mutex);
    if (!st.ready.load(std::memory_order_relaxed)) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
            (void)hipGetLastError();
            set_error("cannot query device %d", dev);
            return MUON_AMD_EDEVICE;
        }
        if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
            set_error("device %d is %s: this library holds gfx950 (MI355X) code only", dev, prop.gcnArchName);
            return MUON_AMD_EDEVICE;
        }
        int rc = raise_lds_limit<Cfg0, false, false>();
        if (rc == MUON_AMD_OK) rc = raise_lds_limit<Cfg0, false, true>();
        if (rc == MUON_AMD_OK) rc = raise_lds_limit<Cfg0, true, true>();
        if (rc == MUON_AMD_OK) rc = raise_lds_limit<Cfg1, false, false>();
        if (rc == MUON_AMD_OK) rc = raise_lds_limit<Cfg1, false, true>();
        if (rc == MUON_AMD_OK) rc = raise_lds_limit<Cfg1, true, true>();
        if (rc != MUON_AMD_OK) return rc;
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) {
            (void)hipGetLastError();
            set_error("cannot look up the static scratch array on device %d", dev);
            return MUON_AMD_ELAUNCH;
        }
        st.scratch_ptr = static_cast<unsigned char*>(ptr);
        st.num_cus = prop.multiProcessorCount;
        st.ready.store(true, std::memory_order_release);
    }
    *out = &st;
    return MUON_AMD_OK;
}

struct ApplyLaunch {            // the fused parameter step of the last update product, or mats == nullptr
    const MuonMatDesc* mats;
    float neg_lr, wd_factor;
    const float* scalars;
};

template <typename Cfg>
static int launch_gemm(const DeviceState& st, const MuonGemmDesc* descs, const MuonTileJob* jobs, int njobs,
                       float alpha, float beta, float gamma, int flags, float* split_partials,
                       int32_t* split_counters, const ApplyLaunch& ap, hipStream_t s) {
    // as many workgroups as the GPU holds at once; each walks its share of the job list
    const int resident = st.num_cus * Cfg::MINB;
    const int grid = njobs < resident ? njobs : resident;
    if (ap.mats)
        hipLaunchKernelGGL((ns_gemm_kernel<Cfg, true, true>), dim3(grid), dim3(Cfg::NT), Cfg::LDS_BYTES, s, descs, jobs,
                           njobs, alpha, beta, gamma, flags, split_partials, split_counters, ap.mats, ap.neg_lr,
                           ap.wd_factor, ap.scalars);
    else if (flags & MUON_AMD_GEMM_Q_KMAJOR)
        hipLaunchKernelGGL((ns_gemm_kernel<Cfg, false, true>), dim3(grid), dim3(Cfg::NT), Cfg::LDS_BYTES, s, descs, jobs,
                           njobs, alpha, beta, gamma, flags, split_partials, split_counters, ap.mats, ap.neg_lr,
                           ap.wd_factor, ap.scalars);
    else
        hipLaunchKernelGGL((ns_gemm_kernel<Cfg, false, false>), dim3(grid), dim3(Cfg::NT), Cfg::LDS_BYTES, s, descs, jobs,
                           njobs, alpha, beta, gamma, flags, split_partials, split_counters, ap.mats, ap.neg_lr,
                           ap.wd_factor, ap.scalars);
    return check_launch("ns_gemm");
}

static int launch_gemm_class(const DeviceState& st, int tile_class, const MuonGemmDesc* descs,
                             const MuonTileJob* jobs, int njobs, float alpha, float beta, float gamma,
                             int flags, float* split_partials, int32_t* split_counters, const ApplyLaunch& ap,
                             hipStream_t s) {
    if (tile_class == 0)
        return launch_gemm<Cfg0>(st, descs, jobs, njobs, alpha, beta, gamma, flags, split_partials, split_counters, ap, s);
    return launch_gemm<Cfg1>(st, descs, jobs, njobs, alpha, beta, gamma, flags, split_partials, split_counters, ap, s);
}

__global__ __launch_bounds__(256) void zero_i32_kernel(int32_t* __restrict__ p, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0;
}

}  // namespace muon_amd

using namespace muon_amd;

extern "C" {

int muon_amd_init(void) {
    const DeviceState* st = nullptr;
    return device_setup(&st);
}

int muon_amd_gemm_tile_rows(int tile_class) {
    MUON_REQUIRE(tile_class >= 0 && tile_class < kNumTileClasses, "gemm_tile_rows: unknown tile class %d", tile_class);
    return kTileClasses[tile_class].bm;
}

int muon_amd_gemm_tile_cols(int tile_class) {
    MUON_REQUIRE(tile_class >= 0 && tile_class < kNumTileClasses, "gemm_tile_cols: unknown tile class %d", tile_class);
    return kTileClasses[tile_class].bn;
}

int muon_amd_validate_gemm(const MuonGemmDesc* descs, int ndesc, const MuonTileJob* jobs,
                           int njobs, int tile_class, int split_slots) {
    MUON_REQUIRE(descs && jobs, "validate_gemm: null table");
    MUON_REQUIRE(split_slots >= 0, "validate_gemm: split_slots=%d", split_slots);
    std::vector<int64_t> covered(static_cast<size_t>(split_slots), 0);   // per split group: K covered, jobs seen
    std::vector<int> seen(static_cast<size_t>(split_slots), 0);
    MUON_REQUIRE(tile_class >= 0 && tile_class < kNumTileClasses, "validate_gemm: unknown tile class %d", tile_class);
    MUON_REQUIRE(ndesc > 0 && njobs > 0, "validate_gemm: ndesc=%d njobs=%d", ndesc, njobs);
    const int TR = kTileClasses[tile_class].bm, TC = kTileClasses[tile_class].bn;
    for (int i = 0; i < ndesc; ++i) {
        const MuonGemmDesc& d = descs[i];
        MUON_REQUIRE(d.P && d.Q, "gemm desc %d: null operand", i);
        MUON_REQUIRE(d.C || d.CT, "gemm desc %d: no output", i);
        MUON_REQUIRE(d.K > 0 && d.K % BK == 0, "gemm desc %d: K=%d is not a positive multiple of %d", i, d.K, BK);
        MUON_REQUIRE(d.rows > 0 && d.colsn > 0 && d.rows % TR == 0 && d.colsn % TC == 0,
                     "gemm desc %d: output %dx%d is not in tiles of %dx%d", i, d.rows, d.colsn, TR, TC);
        MUON_REQUIRE(d.q_kmajor == 0 || d.q_kmajor == 1, "gemm desc %d: q_kmajor=%d", i, d.q_kmajor);
        MUON_REQUIRE(d.q_kmajor == descs[0].q_kmajor, "gemm desc %d: one launch takes its second operands in one layout", i);
        MUON_REQUIRE(d.ldp >= d.K && d.ldq >= (d.q_kmajor ? d.colsn : d.K) && d.ldp % 8 == 0 && d.ldq % 8 == 0,
                     "gemm desc %d: ldp=%d ldq=%d K=%d cols %d (second operand %s)", i, d.ldp, d.ldq, d.K, d.colsn,
                     d.q_kmajor ? "k-major" : "row-major");
        {   // operands and addend are addressed with 32-bit byte offsets from their base pointers
            const int64_t lim = int64_t(1) << 32;
            const int64_t pb = static_cast<int64_t>(d.rows) * d.ldp * 2, db = static_cast<int64_t>(d.rows) * d.ldd * 2;
            const int64_t qb = static_cast<int64_t>(d.q_kmajor ? d.K : d.colsn) * d.ldq * 2;
            MUON_REQUIRE(pb < lim && qb < lim && (!d.D || db < lim),
                         "gemm desc %d: an operand of %lld bytes is beyond the 4 GiB a transfer can address", i,
                         static_cast<long long>(pb > qb ? pb : qb));
        }
        MUON_REQUIRE(!d.q_kmajor || !(d.C && (d.C == d.Q || d.C2 == d.Q)),
                     "gemm desc %d: a k-major second operand is read by every tile of its column block and cannot be overwritten in place", i);
        MUON_REQUIRE(!d.D || (d.ldd >= d.colsn && d.ldd % 8 == 0), "gemm desc %d: ldd=%d cols %d", i, d.ldd, d.colsn);
        MUON_REQUIRE(!(d.C || d.C2) || (d.ldc >= d.colsn && d.ldc % 8 == 0), "gemm desc %d: ldc=%d cols %d", i, d.ldc, d.colsn);
        MUON_REQUIRE(!(d.CT || d.C2T) || (d.ldct >= d.rows && d.ldct % 8 == 0),
                     "gemm desc %d: ldct=%d rows=%d", i, d.ldct, d.rows);
        MUON_REQUIRE((reinterpret_cast<uintptr_t>(d.P) % 16) == 0 && (reinterpret_cast<uintptr_t>(d.Q) % 16) == 0 &&
                         (reinterpret_cast<uintptr_t>(d.C) % 16) == 0 && (reinterpret_cast<uintptr_t>(d.C2) % 16) == 0 &&
                         (reinterpret_cast<uintptr_t>(d.CT) % 16) == 0 && (reinterpret_cast<uintptr_t>(d.C2T) % 16) == 0 &&
                         (reinterpret_cast<uintptr_t>(d.D) % 16) == 0,
                     "gemm desc %d: misaligned pointer", i);
        MUON_REQUIRE(!(d.C2 && !d.C) && !(d.C2T && !d.CT), "gemm desc %d: scaled copy needs its primary output", i);
        MUON_REQUIRE(!d.rowsum || (d.C && d.CT == d.C && !d.D && d.colsn % 64 == 0 && d.ld_rowsum >= d.colsn / 64 &&
                                   (reinterpret_cast<uintptr_t>(d.rowsum) % 4) == 0),
                     "gemm desc %d: row sums need a mirrored product without addend and %d slots per row (ld_rowsum=%d)",
                     i, d.colsn / 64, d.ld_rowsum);
    }
    for (int j = 0; j < njobs; ++j) {
        const MuonTileJob& t = jobs[j];
        MUON_REQUIRE(t.desc >= 0 && t.desc < ndesc, "job %d: desc %d out of range", j, t.desc);
        const MuonGemmDesc& d = descs[t.desc];
        MUON_REQUIRE(t.i0 >= 0 && t.j0 >= 0 && t.i0 % TR == 0 && t.j0 % TC == 0 && t.i0 + TR <= d.rows &&
                         t.j0 + TC <= d.colsn,
                     "job %d: tile (%d,%d) outside %dx%d", j, t.i0, t.j0, d.rows, d.colsn);
        MUON_REQUIRE(t.diag == 0 || t.diag == 1, "job %d: diag=%d", j, t.diag);
        MUON_REQUIRE(t.k0 >= 0 && t.k0 < t.k1 && t.k1 <= d.K && t.k0 % BK == 0 && t.k1 % BK == 0,
                     "job %d: K range %d..%d of %d", j, t.k0, t.k1, d.K);
        const int count = t.split >> 16, idx = t.split & 0xffff;
        if (count <= 1) {
            MUON_REQUIRE(t.split == 0 && t.k0 == 0 && t.k1 == d.K, "job %d: an unsplit job covers all of K", j);
        } else {
            MUON_REQUIRE(kTileClasses[tile_class].split_k, "job %d: tile class %d does not split reductions", j, tile_class);
            MUON_REQUIRE(idx < count && t.part_base >= 0 && t.part_base + count <= split_slots,
                         "job %d: split %d of %d at slot %d, %d slots", j, idx, count, t.part_base, split_slots);
            covered[t.part_base] += t.k1 - t.k0;
            seen[t.part_base] += 1;
            if (seen[t.part_base] == count)
                MUON_REQUIRE(covered[t.part_base] == d.K, "job %d: its split group covers %lld of K=%d", j,
                             static_cast<long long>(covered[t.part_base]), d.K);
            MUON_REQUIRE(seen[t.part_base] <= count, "job %d: split group at slot %d has too many jobs", j, t.part_base);
        }
        // mirrored GEMM: only tiles whose column block is on or above the row block, and tiles
        // inside a diagonal TR x TR block (stored directly, never mirrored) are flagged
        const int cblk = t.j0 / TR * TR;
        MUON_REQUIRE(!(d.CT == d.C && d.C) || (cblk >= t.i0 && t.diag == (cblk == t.i0)),
                     "job %d: mirrored GEMM needs its column block >= row block and diag set on the diagonal block", j);
    }
    for (int g = 0; g < split_slots; ++g)
        MUON_REQUIRE(seen[g] == 0 || covered[g] > 0, "split group %d is inconsistent", g);
    return MUON_AMD_OK;
}

int muon_amd_ns_gemm(const MuonGemmDesc* descs_dev, const MuonTileJob* jobs_dev, int njobs,
                     int tile_class, float alpha, float beta, float gamma, int flags,
                     float* split_partials_dev, int32_t* split_counters_dev, void* stream) {
    MUON_REQUIRE(descs_dev && jobs_dev, "ns_gemm: null table");
    MUON_REQUIRE((split_partials_dev == nullptr) == (split_counters_dev == nullptr),
                 "ns_gemm: split partials and counters go together");
    MUON_REQUIRE(njobs > 0, "ns_gemm: njobs=%d", njobs);
    MUON_REQUIRE(tile_class >= 0 && tile_class < kNumTileClasses, "ns_gemm: unknown tile class %d", tile_class);
    const DeviceState* st = nullptr;
    const int rc = device_setup(&st);
    if (rc != MUON_AMD_OK) return rc;
    return launch_gemm_class(*st, tile_class, descs_dev, jobs_dev, njobs, alpha, beta, gamma, flags,
                             split_partials_dev, split_counters_dev, ApplyLaunch{nullptr, 0.f, 1.f, nullptr},
                             static_cast<hipStream_t>(stream));
}

int muon_amd_ns_gemm_apply(const MuonGemmDesc* descs_dev, const MuonTileJob* jobs_dev, int njobs,
                           int tile_class, float alpha, float beta, int flags,
                           const MuonMatDesc* mats_dev, float lr, float wd_factor,
                           const float* scalars_dev, void* stream) {
    MUON_REQUIRE(descs_dev && jobs_dev && mats_dev, "ns_gemm_apply: null table");
    MUON_REQUIRE(njobs > 0, "ns_gemm_apply: njobs=%d", njobs);
    MUON_REQUIRE(tile_class >= 0 && tile_class < kNumTileClasses, "ns_gemm_apply: unknown tile class %d", tile_class);
    const DeviceState* st = nullptr;
    const int rc = device_setup(&st);
    if (rc != MUON_AMD_OK) return rc;
    return launch_gemm_class(*st, tile_class, descs_dev, jobs_dev, njobs, alpha, beta, 0.f,
                             flags | MUON_AMD_GEMM_Q_KMAJOR, nullptr, nullptr,
                             ApplyLaunch{mats_dev, -lr, wd_factor, scalars_dev}, static_cast<hipStream_t>(stream));
}

int muon_amd_noalloc_max_split_slots(void) { return kStaticSplitSlots; }

int muon_amd_ns_gemm_noalloc(const MuonGemmDesc* descs_dev, const MuonTileJob* jobs_dev, int njobs,
                             int tile_class, float alpha, float beta, float gamma, int flags,
                             int split_slots, void* stream) {
    MUON_REQUIRE(descs_dev && jobs_dev, "ns_gemm_noalloc: null table");
    MUON_REQUIRE(njobs > 0, "ns_gemm_noalloc: njobs=%d", njobs);
    MUON_REQUIRE(tile_class >= 0 && tile_class < kNumTileClasses, "ns_gemm_noalloc: unknown tile class %d", tile_class);
    MUON_REQUIRE(split_slots >= 0, "ns_gemm_noalloc: split_slots=%d", split_slots);
    MUON_REQUIRE(split_slots <= kStaticSplitSlots,
                 "ns_gemm_noalloc: the job list uses %d split slots, the static scratch holds %d "
                 "(use muon_amd_ns_gemm with a caller-owned workspace)", split_slots, kStaticSplitSlots);
    MUON_REQUIRE(split_slots == 0 || kTileClasses[tile_class].split_k,
                 "ns_gemm_noalloc: tile class %d does not split reductions", tile_class);
    const DeviceState* st = nullptr;
    const int rc = device_setup(&st);
    if (rc != MUON_AMD_OK) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    float* const partials = reinterpret_cast<float*>(st->scratch_ptr);
    int32_t* const counters = reinterpret_cast<int32_t*>(st->scratch_ptr + kStaticCounterOffset);
    if (split_slots > 0) {
        // The array keeps whatever the last call left: the counters must start at zero.  A small
        // fill kernel rather than a memset node, so that the call can be recorded into a HIP graph.
        hipLaunchKernelGGL(zero_i32_kernel, dim3((split_slots + 255) / 256), dim3(256), 0, s, counters, split_slots);
        const int zrc = check_launch("ns_gemm_noalloc: clear counters");
        if (zrc != MUON_AMD_OK) return zrc;
    }
    return launch_gemm_class(*st, tile_class, descs_dev, jobs_dev, njobs, alpha, beta, gamma, flags,
                             split_slots > 0 ? partials : nullptr, split_slots > 0 ? counters : nullptr,
                             ApplyLaunch{nullptr, 0.f, 1.f, nullptr}, s);
}

}  // extern "C"
