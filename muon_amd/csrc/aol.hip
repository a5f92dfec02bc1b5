// AOL rescaling of the 4-iteration Newton-Schulz variant (reference muon.py:776-785): from the
// Gram matrix A = X X^T of the un-normalised bf16 matrix X (m x n, m <= n),
//     s_i = max(sum_j |A_ij|, eps),  r_i = s_i^-1/2,
//     X  <- diag(r) X        (both stored orientations),
//     A  <- diag(r) A diag(r)   (the Gram matrix of the rescaled X, so the first iteration needs
//                                no second X X^T product).
// Both kernels are HBM-bound row streams: one wavefront per row, 16-byte accesses.
#include "common.h"

namespace muon_amd {

constexpr int AOL_ROWS_PER_BLOCK = 4;        // one wavefront each
constexpr int AOL_THREADS = AOL_ROWS_PER_BLOCK * 64;

typedef uint32_t u32x4a __attribute__((ext_vector_type(4)));
typedef float f32x4a __attribute__((ext_vector_type(4)));

__device__ __forceinline__ u32x4a ld16(const uint16_t* p) {
    return *(const __attribute__((address_space(1))) u32x4a*)(p);
}
__device__ __forceinline__ void st16(uint16_t* p, u32x4a v) {
    *(__attribute__((address_space(1))) u32x4a*)(p) = v;
}
__device__ __forceinline__ float lo_bf(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float hi_bf(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// r_i = rsqrt(max(bf16(sum_j |A_ij|), eps)): the row sum of a bf16 tensor is a bf16 tensor
// (muon.py:779-781), the rest is fp32.
__global__ __launch_bounds__(AOL_THREADS) void aol_rowsum_kernel(
    const MuonAolDesc* __restrict__ descs, const int32_t* __restrict__ prefix, int nmat, float eps) {
    const int b = blockIdx.x;
    const int mi = find_segment(prefix, nmat, b);
    const MuonAolDesc d = descs[mi];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = (b - prefix[mi]) * AOL_ROWS_PER_BLOCK + wave;      // < m_p by construction
    const uint16_t* __restrict__ a = d.gram + static_cast<int64_t>(row) * d.ld_m;
    float s = 0.f;
    for (int c = lane * 8; c < d.m_p; c += 64 * 8) {
        const u32x4a v = ld16(a + c);
#pragma unroll
        for (int k = 0; k < 4; ++k) s += fabsf(lo_bf(v[k])) + fabsf(hi_bf(v[k]));
    }
    s = wave_sum(s);
    if (lane == 0) d.rvec[row] = rsqrtf(fmaxf(round_bf(s), eps));
}

// The same r from the partial row sums that the X X^T launch left (one float per row and 64-column
// slot, MUON_AMD_GEMM_ROWSUM): lane l adds slots l, l + 64, ... in order, then the wavefront's
// butterfly adds the lanes -- a fixed order, whatever else the launch holds.
__global__ __launch_bounds__(AOL_THREADS) void aol_rowsum_finalize_kernel(
    const MuonAolDesc* __restrict__ descs, const int32_t* __restrict__ prefix, int nmat, float eps) {
    const int b = blockIdx.x;
    const int mi = find_segment(prefix, nmat, b);
    const MuonAolDesc d = descs[mi];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = (b - prefix[mi]) * AOL_ROWS_PER_BLOCK + wave;      // < m_p by construction
    const float* __restrict__ parts = d.rowsum + static_cast<int64_t>(row) * d.ld_rowsum;
    float s = 0.f;
    for (int c = lane; c < d.m_p / 64; c += 64) s += parts[c];
    s = wave_sum(s);
    if (lane == 0) d.rvec[row] = rsqrtf(fmaxf(round_bf(s), eps));
}

// Scales one row of one of the three buffers of a matrix.  Segment 3*mi + 0: rows of X (factor
// r_row), + 1: rows of X^T (factor r_col), + 2: rows of A (factor r_row * r_col).
// rows_only: the rows of A take r_row^2 (A / s, muon.py:785) instead of r_row * r_col.
__global__ __launch_bounds__(AOL_THREADS) void aol_rescale_kernel(
    const MuonAolDesc* __restrict__ descs, const int32_t* __restrict__ prefix, int nmat, int rows_only) {
    const int b = blockIdx.x;
    const int seg = find_segment(prefix, 3 * nmat, b);
    const int mi = seg / 3, kind = seg - 3 * mi;
    const MuonAolDesc d = descs[mi];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = (b - prefix[seg]) * AOL_ROWS_PER_BLOCK + wave;
    const float* __restrict__ r = d.rvec;
    uint16_t* __restrict__ p;
    int width;
    if (kind == 0) {
        p = d.xr + static_cast<int64_t>(row) * d.ld_n;
        width = d.n_p;
    } else if (kind == 1) {
        p = d.xc + static_cast<int64_t>(row) * d.ld_m;
        width = d.m_p;
    } else {
        p = d.gram + static_cast<int64_t>(row) * d.ld_m;
        width = d.m_p;
    }
    const float r_row = (kind == 1) ? 1.f : r[row];
    for (int c = lane * 8; c < width; c += 64 * 8) {
        u32x4a v = ld16(p + c);
        float f[8];
        if (kind == 0) {
#pragma unroll
            for (int k = 0; k < 8; ++k) f[k] = r_row;
        } else if (kind == 2 && rows_only) {
#pragma unroll
            for (int k = 0; k < 8; ++k) f[k] = r_row * r_row;
        } else {
            const f32x4a r0 = *(const __attribute__((address_space(1))) f32x4a*)(r + c);
            const f32x4a r1 = *(const __attribute__((address_space(1))) f32x4a*)(r + c + 4);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                f[k] = r_row * r0[k];
                f[4 + k] = r_row * r1[k];
            }
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = pack2bf(lo_bf(v[k]) * f[2 * k], hi_bf(v[k]) * f[2 * k + 1]);
        st16(p + c, v);
    }
}

}  // namespace muon_amd

using namespace muon_amd;

extern "C" {

int muon_amd_aol_rows_per_block(void) { return AOL_ROWS_PER_BLOCK; }
size_t muon_amd_sizeof_aol_desc(void) { return sizeof(MuonAolDesc); }

int muon_amd_validate_aol(const MuonAolDesc* descs, int nmat, const int32_t* row_prefix,
                          const int32_t* seg_prefix) {
    MUON_REQUIRE(descs && row_prefix && seg_prefix, "validate_aol: null table");
    MUON_REQUIRE(nmat > 0, "validate_aol: nmat=%d", nmat);
    MUON_REQUIRE(row_prefix[0] == 0 && seg_prefix[0] == 0, "validate_aol: prefix must start at 0");
    for (int i = 0; i < nmat; ++i) {
        const MuonAolDesc& d = descs[i];
        MUON_REQUIRE(d.xr && d.gram && d.rvec, "aol desc %d: null pointer", i);
        MUON_REQUIRE(d.m_p > 0 && d.n_p > 0 && d.m_p % 8 == 0 && d.n_p % 8 == 0 &&
                         d.m_p % AOL_ROWS_PER_BLOCK == 0 && d.n_p % AOL_ROWS_PER_BLOCK == 0,
                     "aol desc %d: padded sizes %d x %d", i, d.m_p, d.n_p);
        MUON_REQUIRE(!d.rowsum || (d.m_p % 64 == 0 && d.ld_rowsum >= d.m_p / 64),
                     "aol desc %d: row-sum slots %d for %d rows", i, d.ld_rowsum, d.m_p);
        MUON_REQUIRE(d.ld_n >= d.n_p && d.ld_m >= d.m_p && d.ld_n % 8 == 0 && d.ld_m % 8 == 0,
                     "aol desc %d: leading dimensions %d/%d for %d x %d", i, d.ld_n, d.ld_m, d.m_p, d.n_p);
        MUON_REQUIRE((reinterpret_cast<uintptr_t>(d.xr) % 16) == 0 && (reinterpret_cast<uintptr_t>(d.xc) % 16) == 0 &&
                         (reinterpret_cast<uintptr_t>(d.gram) % 16) == 0 && (reinterpret_cast<uintptr_t>(d.rvec) % 16) == 0,
                     "aol desc %d: pointers must be 16-byte aligned", i);
        MUON_REQUIRE(row_prefix[i + 1] - row_prefix[i] == d.m_p / AOL_ROWS_PER_BLOCK,
                     "aol desc %d: row prefix gives %d blocks, need %d", i, row_prefix[i + 1] - row_prefix[i],
                     d.m_p / AOL_ROWS_PER_BLOCK);
        // (no blocks for the rows of a transposed copy that is not kept)
        const int need[3] = {d.m_p / AOL_ROWS_PER_BLOCK, d.xc ? d.n_p / AOL_ROWS_PER_BLOCK : 0, d.m_p / AOL_ROWS_PER_BLOCK};
        for (int k = 0; k < 3; ++k)
            MUON_REQUIRE(seg_prefix[3 * i + k + 1] - seg_prefix[3 * i + k] == need[k],
                         "aol desc %d: segment %d has %d blocks, need %d", i, k,
                         seg_prefix[3 * i + k + 1] - seg_prefix[3 * i + k], need[k]);
    }
    return MUON_AMD_OK;
}

int muon_amd_aol_rowsum(const MuonAolDesc* descs_dev, const int32_t* row_prefix_dev, int nmat,
                        int nblocks, float eps, void* stream) {
    MUON_REQUIRE(descs_dev && row_prefix_dev, "aol_rowsum: null table");
    MUON_REQUIRE(nmat > 0 && nblocks > 0 && eps > 0.f, "aol_rowsum: nmat=%d nblocks=%d eps=%g", nmat, nblocks, eps);
    hipLaunchKernelGGL(aol_rowsum_kernel, dim3(nblocks), dim3(AOL_THREADS), 0,
                       static_cast<hipStream_t>(stream), descs_dev, row_prefix_dev, nmat, eps);
    return check_launch("aol_rowsum");
}

int muon_amd_aol_rowsum_finalize(const MuonAolDesc* descs_dev, const int32_t* row_prefix_dev, int nmat,
                                 int nblocks, float eps, void* stream) {
    MUON_REQUIRE(descs_dev && row_prefix_dev, "aol_rowsum_finalize: null table");
    MUON_REQUIRE(nmat > 0 && nblocks > 0 && eps > 0.f, "aol_rowsum_finalize: nmat=%d nblocks=%d eps=%g", nmat, nblocks, eps);
    hipLaunchKernelGGL(aol_rowsum_finalize_kernel, dim3(nblocks), dim3(AOL_THREADS), 0,
                       static_cast<hipStream_t>(stream), descs_dev, row_prefix_dev, nmat, eps);
    return check_launch("aol_rowsum_finalize");
}

int muon_amd_aol_rescale(const MuonAolDesc* descs_dev, const int32_t* seg_prefix_dev, int nmat,
                         int nblocks, int mode, void* stream) {
    MUON_REQUIRE(descs_dev && seg_prefix_dev, "aol_rescale: null table");
    MUON_REQUIRE(nmat > 0 && nblocks > 0, "aol_rescale: nmat=%d nblocks=%d", nmat, nblocks);
    MUON_REQUIRE(mode == MUON_AMD_AOL_SYMMETRIC || mode == MUON_AMD_AOL_ROWS_ONLY, "aol_rescale: mode=%d", mode);
    hipLaunchKernelGGL(aol_rescale_kernel, dim3(nblocks), dim3(AOL_THREADS), 0,
                       static_cast<hipStream_t>(stream), descs_dev, seg_prefix_dev, nmat,
                       mode == MUON_AMD_AOL_ROWS_ONLY ? 1 : 0);
    return check_launch("aol_rescale");
}

}  // extern "C"
