// HBM-bound stages of the Muon step for gfx950: momentum/Nesterov/cast, Frobenius norm,
// normalise+transpose, parameter apply, and the auxiliary Adam update.
//
// All launches are "grouped": one launch covers every matrix (tensor) of a chunk.  A block
// finds its matrix by a binary search in a small prefix table and then streams a fixed-size
// contiguous range of it with 16-byte accesses, so a step costs a handful of launches however
// many parameters the model has.
#include "common.h"

namespace muon_amd {

constexpr int EW_THREADS = 256;
constexpr int EW_VEC = 4;                                       // fp32 elements per access
constexpr int EW_ITERS = 8;                                     // accesses in flight per thread and stream
constexpr int EW_PASS_ELEMS = EW_THREADS * EW_VEC * EW_ITERS;   // 8192 elements per pass
#ifndef MUON_EW_PASSES
#define MUON_EW_PASSES 1
#endif
constexpr int EW_PASSES = MUON_EW_PASSES;                       // passes per block (amortise the block's set-up)
constexpr int EW_BLOCK_ELEMS = EW_PASS_ELEMS * EW_PASSES;       // elements per block
constexpr int NT_TILE = 128;                                    // normalise/transposing tile edge

// 16-/8-byte accesses through the global address space (descriptor pointers are generic to the
// compiler).  MUON_EW_NT adds the non-temporal hint to these streaming accesses.
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2e __attribute__((ext_vector_type(2)));
#ifndef MUON_EW_NT
#define MUON_EW_NT 1   // measured +3% on the Llama-3-8B tensors
#endif
__device__ __forceinline__ f32x4 gld4(const float* p) {
#if MUON_EW_NT
    return __builtin_nontemporal_load((const __attribute__((address_space(1))) f32x4*)(p));
#else
    return *(const __attribute__((address_space(1))) f32x4*)(p);
#endif
}
__device__ __forceinline__ void gst4(float* p, f32x4 v) {
#if MUON_EW_NT
    __builtin_nontemporal_store(v, (__attribute__((address_space(1))) f32x4*)(p));
#else
    *(__attribute__((address_space(1))) f32x4*)(p) = v;
#endif
}
__device__ __forceinline__ u32x2e gld2u(const uint16_t* p) {
#if MUON_EW_NT
    return __builtin_nontemporal_load((const __attribute__((address_space(1))) u32x2e*)(p));
#else
    return *(const __attribute__((address_space(1))) u32x2e*)(p);
#endif
}
__device__ __forceinline__ void gst2u(uint16_t* p, u32x2e v) {
#if MUON_EW_NT
    __builtin_nontemporal_store(v, (__attribute__((address_space(1))) u32x2e*)(p));
#else
    *(__attribute__((address_space(1))) u32x2e*)(p) = v;
#endif
}

__device__ __forceinline__ bool aligned_to(const void* p, uintptr_t a) {
    return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

// Storage type of gradients, optimizer state and parameters: fp32, or bf16 (a model kept in
// bf16).  Arithmetic is fp32 either way, as torch's kernels do for bf16 tensors; `rnd` is where
// a value the reference holds in a tensor of the storage type gets that tensor's rounding.
template <typename T>
struct Stored;
template <>
struct Stored<float> {
    static constexpr uintptr_t kAlign = 16;                 // of a 4-element access
    static __device__ __forceinline__ f32x4 ld4(const float* p) { return gld4(p); }
    static __device__ __forceinline__ void st4(float* p, f32x4 v) { gst4(p, v); }
    static __device__ __forceinline__ float ld(const float* p) { return *p; }
    static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
    static __device__ __forceinline__ float rnd(float v) { return v; }
};
template <>
struct Stored<uint16_t> {
    static constexpr uintptr_t kAlign = 8;
    static __device__ __forceinline__ f32x4 ld4(const uint16_t* p) {
        const u32x2e r = gld2u(p);
        return f32x4{__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u),
                     __uint_as_float(r.y << 16), __uint_as_float(r.y & 0xffff0000u)};
    }
    static __device__ __forceinline__ void st4(uint16_t* p, f32x4 v) {
        u32x2e pk;
        pk.x = pack2bf(v[0], v[1]);
        pk.y = pack2bf(v[2], v[3]);
        gst2u(p, pk);
    }
    static __device__ __forceinline__ float ld(const uint16_t* p) { return bf2f(*p); }
    static __device__ __forceinline__ void st(uint16_t* p, float v) { *p = f2bf(v); }
    static __device__ __forceinline__ float rnd(float v) { return round_bf(v); }
};

// Sum of `v` over a 256-thread block, valid in thread 0.
__device__ __forceinline__ float block_sum_256(float v, float* smem4) {
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) smem4[wave] = v;
    __syncthreads();
    return (smem4[0] + smem4[1]) + (smem4[2] + smem4[3]);
}

// ------------------------------------------------------------------------------------------
// momentum: muon.py:9-10 + the bf16 cast of muon.py:277 + partial sums for muon.py:282
// ------------------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float momentum_one(float g, float* m_io, bool has_m, float w,
                                              float beta, int nesterov, float* g_out) {
    if (!has_m) return g;
    const float m_new = Stored<T>::rnd(lerp_torch(*m_io, g, w));      // momentum.lerp_(grad, 1 - beta)
    *m_io = m_new;
    if (!nesterov) return m_new;
    const float u = Stored<T>::rnd(lerp_torch(g, m_new, beta));       // grad.lerp_(momentum, beta)
    *g_out = u;
    return u;
}

// One block's share of a matrix whose gradient and momentum are stored as T.
template <typename T>
__device__ __forceinline__ float momentum_block(const MuonMatDesc& d, int64_t block_base, float w,
                                                float beta, int nesterov, int mutate_grad) {
    const int64_t numel = static_cast<int64_t>(d.rows) * d.cols;
    const bool has_m = d.momentum != nullptr;
    const bool write_g = has_m && nesterov && mutate_grad;
    T* __restrict__ g = static_cast<T*>(d.grad);
    T* __restrict__ mom = static_cast<T*>(d.momentum);
    uint16_t* __restrict__ u = d.u;
    float ss = 0.f;
    const bool aligned = aligned_to(g, Stored<T>::kAlign) && aligned_to(mom, Stored<T>::kAlign) && aligned_to(u, 8);

    for (int pass = 0; pass < EW_PASSES; ++pass) {
        const int64_t base = block_base + static_cast<int64_t>(pass) * EW_PASS_ELEMS;
        if (base >= numel) break;
        if (aligned && base + EW_PASS_ELEMS <= numel) {
            f32x4 gv[EW_ITERS], mv[EW_ITERS];
#pragma unroll
            for (int it = 0; it < EW_ITERS; ++it) {
                const int64_t e = base + (it * EW_THREADS + threadIdx.x) * EW_VEC;
                gv[it] = Stored<T>::ld4(g + e);
                if (has_m) mv[it] = Stored<T>::ld4(mom + e);
                else mv[it] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int it = 0; it < EW_ITERS; ++it) {
                const int64_t e = base + (it * EW_THREADS + threadIdx.x) * EW_VEC;
                f32x4 gg = gv[it], mm = mv[it];
                float uu[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    float gout = gg[k], mk = mm[k];
                    uu[k] = momentum_one<T>(gg[k], &mk, has_m, w, beta, nesterov, &gout);
                    mm[k] = mk;
                    gg[k] = gout;
                    const float ub = round_bf(uu[k]);
                    ss = fmaf(ub, ub, ss);
                }
                if (has_m) Stored<T>::st4(mom + e, mm);
                if (write_g) Stored<T>::st4(g + e, gg);
                u32x2e pk;
                pk.x = pack2bf(uu[0], uu[1]);
                pk.y = pack2bf(uu[2], uu[3]);
                gst2u(u + e, pk);
            }
        } else {
            for (int it = 0; it < EW_ITERS; ++it) {
                const int64_t e0 = base + (it * EW_THREADS + threadIdx.x) * EW_VEC;
#pragma unroll
                for (int k = 0; k < EW_VEC; ++k) {
                    const int64_t e = e0 + k;
                    if (e >= numel) break;
                    const float gval = Stored<T>::ld(g + e);
                    float mval = has_m ? Stored<T>::ld(mom + e) : 0.f;
                    float gout = gval;
                    const float uval = momentum_one<T>(gval, &mval, has_m, w, beta, nesterov, &gout);
                    if (has_m) Stored<T>::st(mom + e, mval);
                    if (write_g) Stored<T>::st(g + e, gout);
                    const uint16_t ub = f2bf(uval);
                    u[e] = ub;
                    const float uf = bf2f(ub);
                    ss = fmaf(uf, uf, ss);
                }
            }
        }
    }
    return ss;
}

// `sc` (optional, device memory): {one_minus_beta, beta} read at run time instead of the by-value
// arguments, so that a captured launch can be replayed with new hyper-parameters.
__global__ __launch_bounds__(EW_THREADS) void momentum_kernel(
    const MuonMatDesc* __restrict__ descs, const int32_t* __restrict__ prefix, int nmat, float w,
    float beta, int nesterov, int mutate_grad, const float* __restrict__ sc) {
    __shared__ float red[4];
    if (sc) {
        w = sc[0];
        beta = sc[1];
    }
    const int b = blockIdx.x;
    const int mi = find_segment(prefix, nmat, b);
    const MuonMatDesc d = descs[mi];
    const int64_t block_base = static_cast<int64_t>(b - prefix[mi]) * EW_BLOCK_ELEMS;
    const float ss = d.src_dtype == MUON_AMD_SRC_BF16
                         ? momentum_block<uint16_t>(d, block_base, w, beta, nesterov, mutate_grad)
                         : momentum_block<float>(d, block_base, w, beta, nesterov, mutate_grad);
    const float total = block_sum_256(ss, red);
    // slot = first slot of the matrix + block within the matrix: the same as the global block id
    // in a launch over the whole table, and still right in a launch over part of it
    if (threadIdx.x == 0) d.partials[d.part_begin + (b - prefix[mi])] = total;
}

// ------------------------------------------------------------------------------------------
// norm finalize: muon.py:282  (X.norm(dim=(-2,-1)) + 1e-7)
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(64) void norm_finalize_kernel(const MuonMatDesc* __restrict__ descs,
                                                            float eps, int round_reference) {
    const MuonMatDesc d = descs[blockIdx.x];
    float s = 0.f;
    for (int i = d.part_begin + threadIdx.x; i < d.part_end; i += 64) s += d.partials[i];
    s = wave_sum(s);
    if (threadIdx.x == 0) {
        float nrm = sqrtf(s);
        float den;
        if (round_reference == 2) {
            den = 1.f;                     // no pre-scale: the AOL variant rescales by rows instead
        } else if (round_reference) {
            nrm = round_bf(nrm);           // the norm of a bf16 tensor is a bf16 tensor
            den = round_bf(nrm + eps);     // bf16 tensor + python scalar -> bf16 tensor
        } else {
            den = nrm + eps;
        }
        *d.denom = den;
    }
}

// ------------------------------------------------------------------------------------------
// normalise (+ transpose) + zero pad:  direct = bf16(u / denom) and / or transp = its transpose;
// an orientation whose pointer is null is not written (the iteration keeps one orientation only:
// the parameter's own for a wide matrix, the transposed one for a tall matrix)
// ------------------------------------------------------------------------------------------
typedef uint32_t u32x4e __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x4e gld4u(const uint16_t* p) {
    return __builtin_nontemporal_load((const __attribute__((address_space(1))) u32x4e*)(p));
}
__device__ __forceinline__ void gst4u(uint16_t* p, u32x4e v) {     // read again soon by the GEMMs: no hint
    *(__attribute__((address_space(1))) u32x4e*)(p) = v;
}

// One NT_TILE x NT_TILE tile per block (256-byte row segments in either orientation; one of the two
// is written: the parameter's own for a wide matrix, the transposed one for a tall matrix).  The
// tile goes through LDS as 32-bit words (two columns each): a thread that later reads word c of
// rows r .. r+7 holds 8 consecutive elements of the two transposed rows 2c and 2c+1.
__global__ __launch_bounds__(256) void normalize_kernel(const MuonMatDesc* __restrict__ descs,
                                                         const int32_t* __restrict__ prefix,
                                                         int nmat) {
    constexpr int PITCH = NT_TILE / 2 + 2;               // words per LDS row (even: 8-byte stores)
    __shared__ __align__(8) uint32_t tile[NT_TILE][PITCH];
    const int b = blockIdx.x;
    const int mi = find_segment(prefix, nmat, b);
    const MuonMatDesc d = descs[mi];
    const int lb = b - prefix[mi];
    const int tiles_c = d.cols_p / NT_TILE;
    const int R0 = (lb / tiles_c) * NT_TILE, C0 = (lb % tiles_c) * NT_TILE;
    const float den = *d.denom;
    const uint16_t* __restrict__ u = d.u;
    const bool vec_ok = (d.cols % 8 == 0) && aligned_to(u, 16);

    constexpr int CH = NT_TILE / 8;                      // 8-element chunks per tile row
    constexpr int NI = NT_TILE * CH / 256;               // chunks per thread
    // every load of the tile goes out before the first result is stored (the stores may alias the
    // loads as far as the compiler knows, so interleaved each load would wait for the store before it)
    u32x4e raws[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int q = threadIdx.x + i * 256;
        const int gr = R0 + q / CH, gc = C0 + (q % CH) * 8;
        raws[i] = u32x4e{0u, 0u, 0u, 0u};
        if (gr < d.rows) {
            const int64_t off = static_cast<int64_t>(gr) * d.cols + gc;
            if (vec_ok && gc + 8 <= d.cols) {
                raws[i] = gld4u(u + off);
            } else {
                uint16_t t[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) t[k] = (gc + k < d.cols) ? u[off + k] : static_cast<uint16_t>(0);
#pragma unroll
                for (int k = 0; k < 4; ++k) raws[i][k] = t[2 * k] | (static_cast<uint32_t>(t[2 * k + 1]) << 16);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int q = threadIdx.x + i * 256;
        const int r = q / CH, cc = (q % CH) * 8;
        const int gr = R0 + r, gc = C0 + cc;
        uint16_t v[8];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            v[2 * k] = static_cast<uint16_t>(raws[i][k] & 0xffffu);
            v[2 * k + 1] = static_cast<uint16_t>(raws[i][k] >> 16);
        }
        if (gr < d.rows) {
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (gc + k < d.cols) v[k] = f2bf(bf2f(v[k]) / den);
        }
        u32x4e o;
#pragma unroll
        for (int k = 0; k < 4; ++k) o[k] = v[2 * k] | (static_cast<uint32_t>(v[2 * k + 1]) << 16);
        if (d.direct) gst4u(d.direct + static_cast<int64_t>(gr) * d.ld_direct + gc, o);
        uint2* const dst = reinterpret_cast<uint2*>(&tile[r][cc / 2]);
        dst[0] = make_uint2(o[0], o[1]);
        dst[1] = make_uint2(o[2], o[3]);
    }
    if (!d.transp) return;                 // (the same for every thread of the block)
    __syncthreads();
#pragma unroll
    for (int i = 0; i < (NT_TILE / 2) * CH / 256; ++i) {
        // work item -> word column c (transposed rows 2c, 2c+1) and source rows r0 .. r0+7
        const int q = threadIdx.x + i * 256;
        const int c = q / CH, r0 = (q % CH) * 8;
        uint32_t w[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) w[k] = tile[r0 + k][c];
        u32x4e lo, hi;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            lo[k] = (w[2 * k] & 0xffffu) | (w[2 * k + 1] << 16);
            hi[k] = (w[2 * k] >> 16) | (w[2 * k + 1] & 0xffff0000u);
        }
        uint16_t* const t = d.transp + static_cast<int64_t>(C0 + 2 * c) * d.ld_transp + R0 + r0;
        gst4u(t, lo);
        gst4u(t + d.ld_transp, hi);
    }
}

// ------------------------------------------------------------------------------------------
// apply: muon.py:14 (aspect scale, in bf16), muon.py:98-99 (decoupled decay + step)
// ------------------------------------------------------------------------------------------
// p.mul_(1 - lr*wd); p.add_(update, alpha=-lr): two tensor operations in the reference, so a
// parameter stored as bf16 is rounded after each (for fp32 storage rnd is the identity).
template <typename T>
__device__ __forceinline__ float apply_one(float p, float us, float neg_lr, float wd_factor) {
    return Stored<T>::rnd(fmaf(neg_lr, us, Stored<T>::rnd(p * wd_factor)));
}

template <typename T>
__device__ __forceinline__ void apply_block(const MuonMatDesc& d, int64_t block_base, float neg_lr,
                                            float wd_factor) {
    const int64_t numel = static_cast<int64_t>(d.rows) * d.cols;
    T* __restrict__ p = static_cast<T*>(d.param);
    uint16_t* __restrict__ out = d.out;
    const uint16_t* __restrict__ res = d.result;
    const float scale = d.scale;
    const bool aligned = (d.cols % 4 == 0) && aligned_to(p, Stored<T>::kAlign) && aligned_to(out, 8);
    for (int pass = 0; pass < EW_PASSES; ++pass) {
        const int64_t base = block_base + static_cast<int64_t>(pass) * EW_PASS_ELEMS;
        if (base >= numel) break;
        if (aligned && base + EW_PASS_ELEMS <= numel) {
            f32x4 pv[EW_ITERS];
            u32x2e ov[EW_ITERS];
#pragma unroll
            for (int it = 0; it < EW_ITERS; ++it) {
                const int64_t e = base + (it * EW_THREADS + threadIdx.x) * EW_VEC;
                const int rr = static_cast<int>(e / d.cols), cc = static_cast<int>(e - static_cast<int64_t>(rr) * d.cols);
                ov[it] = gld2u(res + static_cast<int64_t>(rr) * d.ld_direct + cc);
                if (p) pv[it] = Stored<T>::ld4(p + e);
                else pv[it] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int it = 0; it < EW_ITERS; ++it) {
                const int64_t e = base + (it * EW_THREADS + threadIdx.x) * EW_VEC;
                const float o[4] = {__uint_as_float(ov[it].x << 16), __uint_as_float(ov[it].x & 0xffff0000u),
                                    __uint_as_float(ov[it].y << 16), __uint_as_float(ov[it].y & 0xffff0000u)};
                f32x4 pp = pv[it];
                float us[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    us[k] = round_bf(o[k] * scale);
                    pp[k] = apply_one<T>(pp[k], us[k], neg_lr, wd_factor);
                }
                if (p) Stored<T>::st4(p + e, pp);
                if (out) {
                    u32x2e pk;
                    pk.x = pack2bf(us[0], us[1]);
                    pk.y = pack2bf(us[2], us[3]);
                    gst2u(out + e, pk);
                }
            }
        } else {
            for (int it = 0; it < EW_ITERS; ++it) {
                const int64_t e0 = base + (it * EW_THREADS + threadIdx.x) * EW_VEC;
#pragma unroll
                for (int k = 0; k < EW_VEC; ++k) {
                    const int64_t e = e0 + k;
                    if (e >= numel) break;
                    const int rr = static_cast<int>(e / d.cols), cc = static_cast<int>(e - static_cast<int64_t>(rr) * d.cols);
                    const float us = round_bf(bf2f(res[static_cast<int64_t>(rr) * d.ld_direct + cc]) * scale);
                    if (p) Stored<T>::st(p + e, apply_one<T>(Stored<T>::ld(p + e), us, neg_lr, wd_factor));
                    if (out) out[e] = f2bf(us);
                }
            }
        }
    }
}

// `sc` (optional, device memory): {lr, wd_factor} read at run time instead of the arguments.
__global__ __launch_bounds__(EW_THREADS) void apply_kernel(const MuonMatDesc* __restrict__ descs,
                                                            const int32_t* __restrict__ prefix,
                                                            int nmat, float neg_lr, float wd_factor,
                                                            const float* __restrict__ sc) {
    if (sc) {
        neg_lr = -sc[0];
        wd_factor = sc[1];
    }
    const int b = blockIdx.x;
    const int mi = find_segment(prefix, nmat, b);
    const MuonMatDesc d = descs[mi];
    const int64_t block_base = static_cast<int64_t>(b - prefix[mi]) * EW_BLOCK_ELEMS;
    if (d.src_dtype == MUON_AMD_SRC_BF16) apply_block<uint16_t>(d, block_base, neg_lr, wd_factor);
    else apply_block<float>(d, block_base, neg_lr, wd_factor);
}

// ------------------------------------------------------------------------------------------
// auxiliary Adam: muon.py:104-109 + 257-258
// ------------------------------------------------------------------------------------------
// Every tensor expression of muon.py:105-109 leaves a tensor of the storage type, so for bf16
// storage each of them rounds (grad.square(), both lerps, both bias corrections, the square root,
// "+ eps", the quotient); for fp32 storage rnd is the identity.
template <typename T>
__device__ __forceinline__ float adam_one(float g, float* m, float* v, float w1, float w2,
                                          float eps, float bias1, float bias2) {
    typedef Stored<T> S;
    *m = S::rnd(lerp_torch(*m, g, w1));
    *v = S::rnd(lerp_torch(*v, S::rnd(g * g), w2));
    const float mc = S::rnd(*m / bias1);
    const float vc = S::rnd(*v / bias2);
    return S::rnd(mc / S::rnd(S::rnd(sqrtf(vc)) + eps));
}

template <typename T>
__device__ __forceinline__ void adam_block(const MuonAdamDesc& d, int64_t block_base, float neg_lr,
                                           float wd_factor, float w1, float w2, float eps,
                                           float bias1, float bias2) {
    const int64_t numel = d.numel;
    T* __restrict__ p = static_cast<T*>(d.param);
    const T* __restrict__ g = static_cast<const T*>(d.grad);
    T* __restrict__ m = static_cast<T*>(d.exp_avg);
    T* __restrict__ v = static_cast<T*>(d.exp_avg_sq);
    T* __restrict__ upd = static_cast<T*>(d.update);
    constexpr uintptr_t A = Stored<T>::kAlign;
    const bool aligned = aligned_to(p, A) && aligned_to(g, A) && aligned_to(m, A) && aligned_to(v, A) &&
                         aligned_to(upd, A);
    for (int pass = 0; pass < EW_PASSES; ++pass) {
        const int64_t base = block_base + static_cast<int64_t>(pass) * EW_PASS_ELEMS;
        if (base >= numel) break;
        if (aligned && base + EW_PASS_ELEMS <= numel) {
            f32x4 gv[EW_ITERS], mv[EW_ITERS], vv[EW_ITERS], pv[EW_ITERS];
#pragma unroll
            for (int it = 0; it < EW_ITERS; ++it) {
                const int64_t e = base + (it * EW_THREADS + threadIdx.x) * EW_VEC;
                gv[it] = Stored<T>::ld4(g + e);
                mv[it] = Stored<T>::ld4(m + e);
                vv[it] = Stored<T>::ld4(v + e);
                if (p) pv[it] = Stored<T>::ld4(p + e);
                else pv[it] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int it = 0; it < EW_ITERS; ++it) {
                const int64_t e = base + (it * EW_THREADS + threadIdx.x) * EW_VEC;
                f32x4 mm = mv[it], v2 = vv[it], pp = pv[it], uu;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    float mk = mm[k], vk = v2[k];
                    uu[k] = adam_one<T>(gv[it][k], &mk, &vk, w1, w2, eps, bias1, bias2);
                    mm[k] = mk;
                    v2[k] = vk;
                    pp[k] = apply_one<T>(pp[k], uu[k], neg_lr, wd_factor);
                }
                Stored<T>::st4(m + e, mm);
                Stored<T>::st4(v + e, v2);
                if (p) Stored<T>::st4(p + e, pp);
                if (upd) Stored<T>::st4(upd + e, uu);
            }
        } else {
            // The last, partial pass of a tensor (or a tensor at an odd address): element accesses, four
            // elements at a time with their loads ahead of the arithmetic.  The loop stays rolled: a
            // launch over a few small tensors runs this code once per wave, and what it then waits for
            // is the instruction fetch (unrolled, the pass is several thousand instructions long).
#pragma unroll 1
            for (int it = 0; it < EW_ITERS; ++it) {
                const int64_t e0 = base + (it * EW_THREADS + threadIdx.x) * EW_VEC;
                if (e0 >= numel) break;
                float gs[EW_VEC], ms[EW_VEC], vs[EW_VEC], ps[EW_VEC];
#pragma unroll
                for (int k = 0; k < EW_VEC; ++k) {
                    const int64_t e = e0 + k;
                    const bool in = e < numel;
                    gs[k] = in ? Stored<T>::ld(g + e) : 0.f;
                    ms[k] = in ? Stored<T>::ld(m + e) : 0.f;
                    vs[k] = in ? Stored<T>::ld(v + e) : 0.f;
                    ps[k] = (in && p) ? Stored<T>::ld(p + e) : 0.f;
                }
#pragma unroll
                for (int k = 0; k < EW_VEC; ++k) {
                    const int64_t e = e0 + k;
                    if (e >= numel) continue;
                    float mm = ms[k], v2 = vs[k];
                    const float uu = adam_one<T>(gs[k], &mm, &v2, w1, w2, eps, bias1, bias2);
                    Stored<T>::st(m + e, mm);
                    Stored<T>::st(v + e, v2);
                    if (p) Stored<T>::st(p + e, apply_one<T>(ps[k], uu, neg_lr, wd_factor));
                    if (upd) Stored<T>::st(upd + e, uu);
                }
            }
        }
    }
}

__global__ __launch_bounds__(EW_THREADS) void adam_kernel(const MuonAdamDesc* __restrict__ descs,
                                                           const int32_t* __restrict__ prefix,
                                                           int ntensors, float neg_lr,
                                                           float wd_factor, float w1, float w2,
                                                           float eps, float bias1, float bias2,
                                                           const float* __restrict__ sc) {
    if (sc) {   // {lr, wd_factor, w1, w2, eps, bias1, bias2} read at run time instead of the arguments
        neg_lr = -sc[0];
        wd_factor = sc[1];
        w1 = sc[2];
        w2 = sc[3];
        eps = sc[4];
        bias1 = sc[5];
        bias2 = sc[6];
    }
    const int b = blockIdx.x;
    const int ti = find_segment(prefix, ntensors, b);
    const MuonAdamDesc d = descs[ti];
    const int64_t block_base = static_cast<int64_t>(b - prefix[ti]) * EW_BLOCK_ELEMS;
    if (d.dtype == MUON_AMD_SRC_BF16)
        adam_block<uint16_t>(d, block_base, neg_lr, wd_factor, w1, w2, eps, bias1, bias2);
    else
        adam_block<float>(d, block_base, neg_lr, wd_factor, w1, w2, eps, bias1, bias2);
}

}  // namespace muon_amd

using namespace muon_amd;

extern "C" {

int muon_amd_elementwise_block_elems(void) { return EW_BLOCK_ELEMS; }
int muon_amd_normalize_tile(void) { return NT_TILE; }

int muon_amd_validate_mats(const MuonMatDesc* descs, int nmat, const int32_t* block_prefix,
                           const int32_t* tile_prefix, int tile_edge) {
    MUON_REQUIRE(descs && block_prefix && tile_prefix, "validate_mats: null table");
    MUON_REQUIRE(nmat > 0, "validate_mats: nmat=%d", nmat);
    MUON_REQUIRE(tile_edge > 0 && tile_edge % NT_TILE == 0, "validate_mats: tile_edge=%d", tile_edge);
    MUON_REQUIRE(block_prefix[0] == 0 && tile_prefix[0] == 0, "validate_mats: prefix must start at 0");
    for (int i = 0; i < nmat; ++i) {
        const MuonMatDesc& d = descs[i];
        MUON_REQUIRE(d.rows > 0 && d.cols > 0, "mat %d: rows=%d cols=%d", i, d.rows, d.cols);
        MUON_REQUIRE(d.rows_p >= d.rows && d.cols_p >= d.cols && d.rows_p % tile_edge == 0 &&
                         d.cols_p % tile_edge == 0,
                     "mat %d: padded %dx%d does not cover %dx%d in tiles of %d", i, d.rows_p,
                     d.cols_p, d.rows, d.cols, tile_edge);
        MUON_REQUIRE(d.ld_direct >= d.cols_p && d.ld_transp >= d.rows_p && d.ld_direct % 8 == 0 &&
                         d.ld_transp % 8 == 0,
                     "mat %d: leading dimensions %d/%d for padded %dx%d", i, d.ld_direct, d.ld_transp,
                     d.rows_p, d.cols_p);
        MUON_REQUIRE(d.grad && d.u && (d.direct || d.transp) && d.partials && d.denom,
                     "mat %d: null workspace or source pointer", i);
        MUON_REQUIRE(!d.result || d.result == d.direct,
                     "mat %d: the result of a run without iterations is the normalised matrix in the parameter's orientation", i);
        MUON_REQUIRE(d.param || d.out, "mat %d: neither param nor out given", i);
        MUON_REQUIRE(d.src_dtype == MUON_AMD_SRC_F32 || d.src_dtype == MUON_AMD_SRC_BF16,
                     "mat %d: src_dtype=%d", i, d.src_dtype);
        MUON_REQUIRE((reinterpret_cast<uintptr_t>(d.direct) % 16) == 0 &&
                         (reinterpret_cast<uintptr_t>(d.transp) % 16) == 0 &&
                         (reinterpret_cast<uintptr_t>(d.result) % 16) == 0 &&
                         (reinterpret_cast<uintptr_t>(d.u) % 16) == 0,
                     "mat %d: workspace pointers must be 16-byte aligned", i);
        const int64_t numel = static_cast<int64_t>(d.rows) * d.cols;
        const int64_t nblk = (numel + EW_BLOCK_ELEMS - 1) / EW_BLOCK_ELEMS;
        MUON_REQUIRE(block_prefix[i + 1] - block_prefix[i] == nblk,
                     "mat %d: block prefix gives %d blocks, need %lld", i,
                     block_prefix[i + 1] - block_prefix[i], static_cast<long long>(nblk));
        MUON_REQUIRE(d.part_end - d.part_begin == nblk, "mat %d: partial range %d..%d, need %lld blocks",
                     i, d.part_begin, d.part_end, static_cast<long long>(nblk));
        MUON_REQUIRE(d.part_begin == block_prefix[i], "mat %d: part_begin %d != block prefix %d", i,
                     d.part_begin, block_prefix[i]);
        const int64_t ntile = static_cast<int64_t>(d.rows_p / NT_TILE) * (d.cols_p / NT_TILE);
        MUON_REQUIRE(tile_prefix[i + 1] - tile_prefix[i] == ntile, "mat %d: tile prefix gives %d tiles, need %lld",
                     i, tile_prefix[i + 1] - tile_prefix[i], static_cast<long long>(ntile));
    }
    return MUON_AMD_OK;
}

int muon_amd_momentum(const MuonMatDesc* descs_dev, const int32_t* block_prefix_dev, int nmat,
                      int nblocks, float one_minus_beta, float beta, int nesterov,
                      int mutate_grad, const float* scalars_dev, void* stream) {
    MUON_REQUIRE(descs_dev && block_prefix_dev, "momentum: null table");
    MUON_REQUIRE(nmat > 0 && nblocks > 0, "momentum: nmat=%d nblocks=%d", nmat, nblocks);
    hipLaunchKernelGGL(momentum_kernel, dim3(nblocks), dim3(EW_THREADS), 0,
                       static_cast<hipStream_t>(stream), descs_dev, block_prefix_dev, nmat,
                       one_minus_beta, beta, nesterov, mutate_grad, scalars_dev);
    return check_launch("momentum");
}

int muon_amd_norm_finalize(const MuonMatDesc* descs_dev, int nmat, float eps, int flags,
                           void* stream) {
    MUON_REQUIRE(descs_dev, "norm_finalize: null table");
    MUON_REQUIRE(nmat > 0, "norm_finalize: nmat=%d", nmat);
    hipLaunchKernelGGL(norm_finalize_kernel, dim3(nmat), dim3(64), 0,
                       static_cast<hipStream_t>(stream), descs_dev, eps,
                       (flags & MUON_AMD_NORM_UNIT) ? 2 : ((flags & MUON_AMD_ROUND_REFERENCE) ? 1 : 0));
    return check_launch("norm_finalize");
}

int muon_amd_normalize(const MuonMatDesc* descs_dev, const int32_t* tile_prefix_dev, int nmat,
                       int ntiles, void* stream) {
    MUON_REQUIRE(descs_dev && tile_prefix_dev, "normalize: null table");
    MUON_REQUIRE(nmat > 0 && ntiles > 0, "normalize: nmat=%d ntiles=%d", nmat, ntiles);
    hipLaunchKernelGGL(normalize_kernel, dim3(ntiles), dim3(256), 0,
                       static_cast<hipStream_t>(stream), descs_dev, tile_prefix_dev, nmat);
    return check_launch("normalize");
}

int muon_amd_apply(const MuonMatDesc* descs_dev, const int32_t* block_prefix_dev, int nmat,
                   int nblocks, float lr, float wd_factor, const float* scalars_dev, void* stream) {
    MUON_REQUIRE(descs_dev && block_prefix_dev, "apply: null table");
    MUON_REQUIRE(nmat > 0 && nblocks > 0, "apply: nmat=%d nblocks=%d", nmat, nblocks);
    hipLaunchKernelGGL(apply_kernel, dim3(nblocks), dim3(EW_THREADS), 0,
                       static_cast<hipStream_t>(stream), descs_dev, block_prefix_dev, nmat, -lr,
                       wd_factor, scalars_dev);
    return check_launch("apply");
}

int muon_amd_adam(const MuonAdamDesc* descs_dev, const int32_t* block_prefix_dev, int ntensors,
                  int nblocks, float lr, float wd_factor, float w1, float w2, float eps,
                  float bias1, float bias2, const float* scalars_dev, void* stream) {
    MUON_REQUIRE(descs_dev && block_prefix_dev, "adam: null table");
    MUON_REQUIRE(ntensors > 0 && nblocks > 0, "adam: ntensors=%d nblocks=%d", ntensors, nblocks);
    MUON_REQUIRE(scalars_dev || (bias1 != 0.f && bias2 != 0.f), "adam: zero bias correction");
    hipLaunchKernelGGL(adam_kernel, dim3(nblocks), dim3(EW_THREADS), 0,
                       static_cast<hipStream_t>(stream), descs_dev, block_prefix_dev, ntensors,
                       -lr, wd_factor, w1, w2, eps, bias1, bias2, scalars_dev);
    return check_launch("adam");
}

}  // extern "C"
