// Grouped bf16 MFMA GEMM for the Newton-Schulz iteration on gfx950 (CDNA4).
//
// Every product of the iteration (muon.py:285-287) is computed as an "NT" GEMM
//     acc[i][j] = sum_k P[i][k] * Q[j][k]
// whose two operands are both contiguous along k:
//     A  = X X^T                P = Q = X            (rows of X)
//     A A (A symmetric)         P = A or c*A, Q = A  ((A A)[i][j] = sum_k A[i][k] A[j][k])
//     B X (B symmetric)         P = B, Q = X^T       (X^T kept beside X by the epilogue)
// so one kernel serves all three, and no operand ever needs a transposing load.  The epilogue
// fuses the polynomial terms (b*A + c*A*A, a*X + B*X), writes the tile and its transpose (the
// mirror half of a symmetric result, or X^T for the next iteration), and optionally a scaled
// copy (c*A).  Symmetric results only compute tiles on or above the diagonal.
//
// A launch covers a job list of output tiles drawn from many matrices.  A workgroup computes
// one BM x BN tile with BK = 64: global -> registers -> LDS (double buffered, rows padded by
// 16 bytes so the ds_read_b128 fragment loads are bank-conflict free), then
// v_mfma_f32_32x32x16_bf16 with fp32 accumulation.
#include "common.h"

namespace muon_amd {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// 16-byte load through the global (not flat) address space: pointers fetched from a descriptor
// are generic to the compiler, and a flat load would also count against the LDS wait counter.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u32x4 gload16(const uint16_t* p) {
    return *(const __attribute__((address_space(1))) u32x4*)(p);
}
__device__ __forceinline__ uint16_t gload2(const uint16_t* p) {
    return *(const __attribute__((address_space(1))) uint16_t*)(p);
}
__device__ __forceinline__ void gstore2(uint16_t* p, uint16_t v) {
    *(__attribute__((address_space(1))) uint16_t*)(p) = v;
}
__device__ __forceinline__ void gstore8(uint16_t* p, u32x2 v) {
    *(__attribute__((address_space(1))) u32x2*)(p) = v;
}

constexpr int BK = 64;           // k extent of one LDS stage
constexpr int LDK = BK + 8;      // padded LDS row length in elements (144 bytes)

template <int BM, int BN, int WGM, int WGN>
struct GemmCfg {
    static constexpr int NT = WGM * WGN * 64;
    static constexpr int WM = BM / WGM, WN = BN / WGN;
    static constexpr int TM = WM / 32, TN = WN / 32;
    static constexpr int ROWS_PER_PASS = NT / 8;          // 8 x 16-byte chunks per 64-wide row
    static constexpr int PCH = BM / ROWS_PER_PASS, QCH = BN / ROWS_PER_PASS;
    static constexpr int STAGE = (BM + BN) * LDK;         // elements per LDS stage
    static constexpr size_t LDS_BYTES = 2u * STAGE * sizeof(uint16_t);
    static_assert(BM % (WGM * 32) == 0 && BN % (WGN * 32) == 0, "wave tile must be MFMA tiles");
    static_assert(BM % ROWS_PER_PASS == 0 && BN % ROWS_PER_PASS == 0, "loader must tile the stage");
};

template <int BM, int BN, int WGM, int WGN, int MINB>
__global__ __launch_bounds__(WGM * WGN * 64, MINB) void ns_gemm_kernel(
    const MuonGemmDesc* __restrict__ descs, const MuonTileJob* __restrict__ jobs, float alpha,
    float beta, float gamma, int round_terms) {
    using Cfg = GemmCfg<BM, BN, WGM, WGN>;
    constexpr int NT = Cfg::NT, TM = Cfg::TM, TN = Cfg::TN, PCH = Cfg::PCH, QCH = Cfg::QCH;
    extern __shared__ __align__(16) uint16_t lds[];

    const MuonTileJob job = jobs[blockIdx.x];
    const MuonGemmDesc d = descs[job.desc];
    const int i0 = job.i0, j0 = job.j0;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;

    // ---- global -> register -> LDS staging --------------------------------------------------
    const int crow = tid >> 3, cchunk = (tid & 7) * 8;
    const uint16_t* __restrict__ Pg = d.P + static_cast<size_t>(i0 + crow) * d.ldp + cchunk;
    const uint16_t* __restrict__ Qg = d.Q + static_cast<size_t>(j0 + crow) * d.ldq + cchunk;
    const size_t pstep = static_cast<size_t>(Cfg::ROWS_PER_PASS) * d.ldp;
    const size_t qstep = static_cast<size_t>(Cfg::ROWS_PER_PASS) * d.ldq;
    uint16_t* const lds_p = lds + crow * LDK + cchunk;
    uint16_t* const lds_q = lds + (BM + crow) * LDK + cchunk;

    u32x4 pr[PCH], qr[QCH];
    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;

    // fragment read offsets: lane l reads row (l % 32), k offset (l / 32) * 8 of each 32 x 16 slab
    const int frag_off = (lane & 31) * LDK + (lane >> 5) * 8;
    const uint16_t* const lds_pw = lds + (wm * Cfg::WM) * LDK + frag_off;
    const uint16_t* const lds_qw = lds + (BM + wn * Cfg::WN) * LDK + frag_off;

#define NS_GLOAD(kb_)                                                                       \
    do {                                                                                    \
        _Pragma("unroll") for (int i_ = 0; i_ < PCH; ++i_) pr[i_] =                         \
            gload16(Pg + i_ * pstep + static_cast<size_t>(kb_) * BK);                       \
        _Pragma("unroll") for (int i_ = 0; i_ < QCH; ++i_) qr[i_] =                         \
            gload16(Qg + i_ * qstep + static_cast<size_t>(kb_) * BK);                       \
    } while (0)
#define NS_LSTORE(stage_)                                                                   \
    do {                                                                                    \
        _Pragma("unroll") for (int i_ = 0; i_ < PCH; ++i_) *reinterpret_cast<u32x4*>(       \
            lds_p + (stage_) * Cfg::STAGE + i_ * Cfg::ROWS_PER_PASS * LDK) = pr[i_];        \
        _Pragma("unroll") for (int i_ = 0; i_ < QCH; ++i_) *reinterpret_cast<u32x4*>(       \
            lds_q + (stage_) * Cfg::STAGE + i_ * Cfg::ROWS_PER_PASS * LDK) = qr[i_];        \
    } while (0)
#define NS_COMPUTE(stage_)                                                                  \
    do {                                                                                    \
        const uint16_t* ps_ = lds_pw + (stage_) * Cfg::STAGE;                               \
        const uint16_t* qs_ = lds_qw + (stage_) * Cfg::STAGE;                               \
        _Pragma("unroll") for (int ks_ = 0; ks_ < BK / 16; ++ks_) {                         \
            bf16x8 af_[TM], bf_[TN];                                                        \
            _Pragma("unroll") for (int a_ = 0; a_ < TM; ++a_) af_[a_] =                     \
                *reinterpret_cast<const bf16x8*>(ps_ + a_ * 32 * LDK + ks_ * 16);           \
            _Pragma("unroll") for (int b_ = 0; b_ < TN; ++b_) bf_[b_] =                     \
                *reinterpret_cast<const bf16x8*>(qs_ + b_ * 32 * LDK + ks_ * 16);           \
            _Pragma("unroll") for (int a_ = 0; a_ < TM; ++a_)                               \
                _Pragma("unroll") for (int b_ = 0; b_ < TN; ++b_) acc[a_][b_] =             \
                    __builtin_amdgcn_mfma_f32_32x32x16_bf16(af_[a_], bf_[b_], acc[a_][b_],  \
                                                            0, 0, 0);                       \
        }                                                                                   \
    } while (0)

    const int nk = d.K / BK;
    NS_GLOAD(0);
    NS_LSTORE(0);
    __syncthreads();
    int cur = 0;
    for (int kb = 1; kb < nk; ++kb) {
        NS_GLOAD(kb);              // next k-block: in flight while the current one is multiplied
        __builtin_amdgcn_sched_barrier(0);   // keep the loads ahead of the MFMA block
        NS_COMPUTE(cur);
        __builtin_amdgcn_sched_barrier(0);
        NS_LSTORE(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }
    NS_COMPUTE(cur);
#undef NS_GLOAD
#undef NS_LSTORE
#undef NS_COMPUTE

    // ---- epilogue ------------------------------------------------------------------------------
    // acc[a][b][i] is output (row, col) = (rb + 8*(i/4) + (i%4), cb) with
    //   rb = i0 + wm*WM + a*32 + 4*(lane/32),  cb = j0 + wn*WN + b*32 + lane%32.
    const bool mirror_ok = !(job.diag && d.CT == d.C);
    const uint16_t* D = d.D;   // may alias C (in-place a*X + B*X): no restrict
#pragma unroll
    for (int a = 0; a < TM; ++a) {
#pragma unroll
        for (int b = 0; b < TN; ++b) {
            const int cb = j0 + wn * Cfg::WN + b * 32 + (lane & 31);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int rb = i0 + wm * Cfg::WM + a * 32 + 8 * q + 4 * (lane >> 5);
                float o[4], o2[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float t1 = alpha * acc[a][b][4 * q + e];
                    float t2 = 0.f;
                    if (D) t2 = beta * bf2f(gload2(D + static_cast<size_t>(rb + e) * d.ldd + cb));
                    if (round_terms) {
                        t1 = round_bf(t1);
                        t2 = round_bf(t2);
                    }
                    o[e] = round_bf(t1 + t2);
                    o2[e] = gamma * o[e];
                }
                if (d.C) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        gstore2(d.C + static_cast<size_t>(rb + e) * d.ldc + cb, f2bf(o[e]));
                }
                if (d.C2) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        gstore2(d.C2 + static_cast<size_t>(rb + e) * d.ldc + cb, f2bf(o2[e]));
                }
                if (mirror_ok) {
                    if (d.CT) {
                        u32x2 pk;
                        pk.x = pack2bf(o[0], o[1]);
                        pk.y = pack2bf(o[2], o[3]);
                        gstore8(d.CT + static_cast<size_t>(cb) * d.ldct + rb, pk);
                    }
                    if (d.C2T) {
                        u32x2 pk;
                        pk.x = pack2bf(o2[0], o2[1]);
                        pk.y = pack2bf(o2[2], o2[3]);
                        gstore8(d.C2T + static_cast<size_t>(cb) * d.ldct + rb, pk);
                    }
                }
            }
        }
    }
}

struct TileClass {
    int edge;
    int threads;
    size_t lds_bytes;
};

static const TileClass kTileClasses[2] = {
    {128, GemmCfg<128, 128, 2, 2>::NT, GemmCfg<128, 128, 2, 2>::LDS_BYTES},
    {256, GemmCfg<256, 256, 2, 4>::NT, GemmCfg<256, 256, 2, 4>::LDS_BYTES},
};

}  // namespace muon_amd

using namespace muon_amd;

extern "C" {

int muon_amd_gemm_tile(int tile_class) {
    MUON_REQUIRE(tile_class == 0 || tile_class == 1, "gemm_tile: unknown tile class %d", tile_class);
    return kTileClasses[tile_class].edge;
}

int muon_amd_validate_gemm(const MuonGemmDesc* descs, int ndesc, const MuonTileJob* jobs,
                           int njobs, int tile_class) {
    MUON_REQUIRE(descs && jobs, "validate_gemm: null table");
    MUON_REQUIRE(tile_class == 0 || tile_class == 1, "validate_gemm: unknown tile class %d", tile_class);
    MUON_REQUIRE(ndesc > 0 && njobs > 0, "validate_gemm: ndesc=%d njobs=%d", ndesc, njobs);
    const int T = kTileClasses[tile_class].edge;
    for (int i = 0; i < ndesc; ++i) {
        const MuonGemmDesc& d = descs[i];
        MUON_REQUIRE(d.P && d.Q, "gemm desc %d: null operand", i);
        MUON_REQUIRE(d.C || d.CT, "gemm desc %d: no output", i);
        MUON_REQUIRE(d.K > 0 && d.K % BK == 0, "gemm desc %d: K=%d is not a positive multiple of %d", i, d.K, BK);
        MUON_REQUIRE(d.rows > 0 && d.colsn > 0 && d.rows % T == 0 && d.colsn % T == 0,
                     "gemm desc %d: output %dx%d is not in tiles of %d", i, d.rows, d.colsn, T);
        MUON_REQUIRE(d.ldp >= d.K && d.ldq >= d.K && d.ldp % 8 == 0 && d.ldq % 8 == 0,
                     "gemm desc %d: ldp=%d ldq=%d K=%d", i, d.ldp, d.ldq, d.K);
        MUON_REQUIRE(!d.D || (d.ldd >= d.colsn), "gemm desc %d: ldd=%d < cols %d", i, d.ldd, d.colsn);
        MUON_REQUIRE(!(d.C || d.C2) || d.ldc >= d.colsn, "gemm desc %d: ldc=%d < cols %d", i, d.ldc, d.colsn);
        MUON_REQUIRE(!(d.CT || d.C2T) || (d.ldct >= d.rows && d.ldct % 4 == 0),
                     "gemm desc %d: ldct=%d rows=%d", i, d.ldct, d.rows);
        MUON_REQUIRE((reinterpret_cast<uintptr_t>(d.P) % 16) == 0 && (reinterpret_cast<uintptr_t>(d.Q) % 16) == 0 &&
                         (reinterpret_cast<uintptr_t>(d.CT) % 8) == 0 && (reinterpret_cast<uintptr_t>(d.C2T) % 8) == 0,
                     "gemm desc %d: misaligned pointer", i);
        MUON_REQUIRE(!(d.C2 && !d.C) && !(d.C2T && !d.CT), "gemm desc %d: scaled copy needs its primary output", i);
    }
    for (int j = 0; j < njobs; ++j) {
        const MuonTileJob& t = jobs[j];
        MUON_REQUIRE(t.desc >= 0 && t.desc < ndesc, "job %d: desc %d out of range", j, t.desc);
        const MuonGemmDesc& d = descs[t.desc];
        MUON_REQUIRE(t.i0 >= 0 && t.j0 >= 0 && t.i0 % T == 0 && t.j0 % T == 0 && t.i0 + T <= d.rows &&
                         t.j0 + T <= d.colsn,
                     "job %d: tile (%d,%d) outside %dx%d", j, t.i0, t.j0, d.rows, d.colsn);
        MUON_REQUIRE(t.diag == 0 || t.diag == 1, "job %d: diag=%d", j, t.diag);
        MUON_REQUIRE(!(d.CT == d.C && d.C) || (t.j0 >= t.i0 && t.diag == (t.i0 == t.j0)),
                     "job %d: mirrored GEMM needs j0 >= i0 and diag set on the diagonal", j);
    }
    return MUON_AMD_OK;
}

int muon_amd_ns_gemm(const MuonGemmDesc* descs_dev, const MuonTileJob* jobs_dev, int njobs,
                     int tile_class, float alpha, float beta, float gamma, int flags,
                     void* stream) {
    MUON_REQUIRE(descs_dev && jobs_dev, "ns_gemm: null table");
    MUON_REQUIRE(njobs > 0, "ns_gemm: njobs=%d", njobs);
    MUON_REQUIRE(tile_class == 0 || tile_class == 1, "ns_gemm: unknown tile class %d", tile_class);
    const int rt = (flags & MUON_AMD_ROUND_REFERENCE) ? 1 : 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (tile_class == 0) {
        auto kern = ns_gemm_kernel<128, 128, 2, 2, 2>;
        static bool attr_set = false;
        if (!attr_set) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    static_cast<int>(kTileClasses[0].lds_bytes)) != hipSuccess) {
                set_error("ns_gemm: cannot raise dynamic LDS to %zu bytes", kTileClasses[0].lds_bytes);
                return MUON_AMD_ELAUNCH;
            }
            attr_set = true;
        }
        hipLaunchKernelGGL(kern, dim3(njobs), dim3(kTileClasses[0].threads), kTileClasses[0].lds_bytes, s,
                           descs_dev, jobs_dev, alpha, beta, gamma, rt);
    } else {
        auto kern = ns_gemm_kernel<256, 256, 2, 4, 1>;
        static bool attr_set = false;
        if (!attr_set) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    static_cast<int>(kTileClasses[1].lds_bytes)) != hipSuccess) {
                set_error("ns_gemm: cannot raise dynamic LDS to %zu bytes", kTileClasses[1].lds_bytes);
                return MUON_AMD_ELAUNCH;
            }
            attr_set = true;
        }
        hipLaunchKernelGGL(kern, dim3(njobs), dim3(kTileClasses[1].threads), kTileClasses[1].lds_bytes, s,
                           descs_dev, jobs_dev, alpha, beta, gamma, rt);
    }
    return check_launch("ns_gemm");
}

}  // extern "C"
