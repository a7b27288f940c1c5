// Device-side building blocks shared by the deformable-convolution kernels (gfx950 / CDNA4).
//
//  * Mma<T>      -- one MFMA tile per data type: v_mfma_f32_32x32x2_f32 for float,
//                   v_mfma_f64_16x16x4_f64 for double, with the register->row map of the result.
//  * TapGeo      -- the sampling geometry of one (kernel tap, output position): inside test,
//                   corner offsets and fractions, following the reference sampler
//                   (deform3d/lib/deform_conv3d_cuda_kernel.cu:21-26,40-45,123-124 and
//                   deform2d_double/lib/deform_conv2d_cuda_kernel.cu:31-34,43-46,114-115).
#pragma once
#include <hip/hip_runtime.h>

namespace dcn {

struct Params {
    int nd;                       // 2 or 3 (informative; kernels are templated on it)
    int N, C_in, C_out, G, cpg, DG;
    int M, Cg;                    // output / input channels per convolution group
    int in[3], out[3], k[3], pad[3], stride[3], dil[3];   // (l,h,w); 2-D uses slots 1,2
    unsigned inV, outV;           // voxels per channel, input / output
    int kV;
    int tiles;                    // position tiles per sample (kernel specific)
    int mchunks;                  // output-channel chunks handled by separate workgroups
    int Mp, Cgp;                  // padded extents of the re-laid-out weight in the workspace
    int nsplit;                   // backward-weight: number of position splits
    int nctiles;                  // backward-weight: channel tiles over all (group, deformable group) segments
    // LDS halo tiling (kernels that stage an input neighbourhood in LDS); slots as in[] / out[]
    int tdim[3];                  // output positions per workgroup tile along each axis
    int ntile[3];                 // tiles along each axis
    int hext[3];                  // halo extent in input voxels along each axis
    int mlo[3];                   // halo margin below the lowest integer tap coordinate
    int hvol;                     // hext[0] * hext[1] * hext[2]
    int hstride;                  // LDS elements between the planes of two channels (>= hvol)
    int cchunk;                   // channels staged per pass
    int oob_zero;                 // 3-D backward: 1 = no grad_offset term for out-of-range samples
};

// Halo margin chosen on the device.  How far the LDS halo of a position block must reach depends on
// the offsets, which the host never sees: a sample whose corners lie outside the halo takes a slow
// path through global memory, and a halo wider than the offsets need costs LDS that the channels
// could have used.  The host therefore plans the halo kernels for up to MAX_PLANS margins (same
// position blocks, so the plans differ in the fields of HaloPlan only); one
// block of the weight-packing kernel that precedes them counts, over a spread of the offsets, how
// many reach past each margin, prices every plan and writes the index of the cheapest to *sel.  A
// kernel launch serves the plans of its `mask` and returns at once when another one was chosen.
constexpr int MAX_PLANS = 3;
struct HaloPlan {                 // what a margin changes in Params
    int hext[3], mlo[3], hvol, hstride, cchunk;
};
struct PlanSet {
    HaloPlan alt[MAX_PLANS - 1];  // plans 1 .. MAX_PLANS - 1 (plan 0 is the Params argument itself)
    unsigned mask;                // bit i: this launch runs plan i
};
// The split units at the end of a forward launch (after `whole` unsplit ones) come in two runs: the
// first unitsA units are split `csplit` ways (the kernel argument), the others splitB ways, with at
// most cchB channels per LDS pass so that their workgroups get equal shares (splitB = 0: one run).
// Their workgroups follow in that order, and so do their partial sums.
struct TailSplit {
    unsigned unitsA;
    int splitB, cchB;
};
struct PlanChoice {
    unsigned* sel;                // chosen plan (device memory), null: a single plan, nothing to choose
    int nplans, nd;
    int margin[MAX_PLANS];        // ascending
    float base[MAX_PLANS];        // cost of the plan when no sample leaves its halo, plan 0 = 1
    // cost added by samples beyond the halo, as a factor 1 + far_wave * P(some lane of a wavefront
    // holds such a sample) + far_sample * p + far_steep * p^8 with p = P(a sample is one): the last
    // term for the scatter, whose global atomics spread over more and more cache lines as the offsets grow
    float far_wave, far_sample, far_steep;
    // > 0: the path without LDS tiling (grad-input by global atomics on a channels-last copy) is on
    // offer as well, at this cost whatever the offsets; it is chosen (*sel = MAX_PLANS) when every
    // halo plan costs more, i.e. when most samples would leave even the widest halo
    float global_cost;
};
// A kernel of a path that the device may or may not have chosen: returns true when *gate names
// another plan (gate == nullptr: not gated).
__device__ inline bool gated_out(const unsigned* __restrict__ gate, unsigned want) {
    return gate && (unsigned)__builtin_amdgcn_readfirstlane((int)*gate) != want;
}
// The halo fields of the chosen plan in H; false when this launch does not serve it (uniform for
// the grid).  Kept apart from P, which stays the kernel argument: its other fields can then be
// re-read from the argument segment wherever they are needed instead of living in registers.
// (field by field from constant argument offsets, no indexed copy)
__device__ inline bool chosen_halo(const Params& P, const PlanSet& S, const unsigned* __restrict__ sel, HaloPlan& H) {
    unsigned idx = 0;
    if (sel) idx = (unsigned)__builtin_amdgcn_readfirstlane((int)*sel);
    if (idx >= (unsigned)MAX_PLANS || !((S.mask >> idx) & 1u)) return false;
    static_assert(MAX_PLANS == 3, "two alternatives are selected between");
    const bool zero = idx == 0, one = idx == 1;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        H.hext[a] = zero ? P.hext[a] : one ? S.alt[0].hext[a] : S.alt[1].hext[a];
        H.mlo[a] = zero ? P.mlo[a] : one ? S.alt[0].mlo[a] : S.alt[1].mlo[a];
    }
    H.hvol = zero ? P.hvol : one ? S.alt[0].hvol : S.alt[1].hvol;
    H.hstride = zero ? P.hstride : one ? S.alt[0].hstride : S.alt[1].hstride;
    H.cchunk = zero ? P.cchunk : one ? S.alt[0].cchunk : S.alt[1].cchunk;
    return true;
}

// ---------------------------------------------------------------------------------------------
template <typename T> struct Mma;

// v_mfma_f32_32x32x2_f32: A is 32x2, B is 2x32, D is 32x32.  Lane l supplies A[l%32][l/32] and
// B[l/32][l%32]; it receives D[row(r, l/32)][l%32] in 16 registers r, rows grouped in fours.
template <> struct Mma<float> {
    static constexpr int TN = 32;     // tile edge (rows of A, columns of B)
    static constexpr int KL = 2;      // reduction slots spread over lane groups
    static constexpr int NACC = 16;
    typedef float Acc __attribute__((ext_vector_type(16)));
    __device__ static inline Acc mma(float a, float b, Acc c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
    __host__ __device__ static constexpr int row(int r, int lg) { return (r >> 2) * 8 + lg * 4 + (r & 3); }
};

// v_mfma_f64_16x16x4_f64: A is 16x4, B is 4x16, D is 16x16.  Lane l supplies A[l%16][l/16] and
// B[l/16][l%16]; it receives D[4*r + l/16][l%16] in 4 registers r.
template <> struct Mma<double> {
    static constexpr int TN = 16;
    static constexpr int KL = 4;
    static constexpr int NACC = 4;
    typedef double Acc __attribute__((ext_vector_type(4)));
    __device__ static inline Acc mma(double a, double b, Acc c) {
        return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
    }
    __host__ __device__ static constexpr int row(int r, int lg) { return r * 4 + lg; }
};

template <typename T> __device__ inline typename Mma<T>::Acc acc_zero() {
    typename Mma<T>::Acc z;
#pragma unroll
    for (int i = 0; i < Mma<T>::NACC; ++i) z[i] = 0;
    return z;
}

// ---------------------------------------------------------------------------------------------
// Axis a of an ND kernel lives in slot a + (3 - ND) of the Params arrays.
template <int ND> __device__ inline constexpr int slot(int a) { return a + 3 - ND; }

template <int ND>
__device__ inline void decode_pos(const Params& P, unsigned pos, int o[ND]) {
    if constexpr (ND == 3) {
        o[2] = pos % P.out[2];
        unsigned t = pos / P.out[2];
        o[1] = t % P.out[1];
        o[0] = t / P.out[1];
    } else {
        o[1] = pos % P.out[2];
        o[0] = pos / P.out[2];
    }
}

template <int ND>
__device__ inline void decode_tap(const Params& P, int tap, int kk[ND]) {
    if constexpr (ND == 3) {
        kk[2] = tap % P.k[2];
        int t = tap / P.k[2];
        kk[1] = t % P.k[1];
        kk[0] = t / P.k[1];
    } else {
        kk[1] = tap % P.k[2];
        kk[0] = tap / P.k[2];
    }
}

template <typename T, int ND>
struct TapGeo {
    static constexpr int NC = 1 << ND;
    unsigned idx[NC];   // voxel offset of each corner inside one channel; corner bit (ND-1-a) = high on axis a
    T f[ND];            // fraction toward the high corner on each axis
    T p[ND];            // absolute sampling coordinate
    int lo[ND], hi[ND]; // low / high corner coordinate per axis
    bool inside;        // strict -1 < p < size on every axis
};

// `offv[a]` is the learned offset of this (tap, position) on axis a, `ib[a]` is out*stride - pad
// of this lane's position, `kd[a]` is tap*dilation (wave-uniform).  Corner indices are only
// meaningful when `inside`; otherwise they are zero so that a masked-off lane never forms a wild
// address.
template <typename T, int ND>
__device__ inline void load_offsets(const Params& P, const T* __restrict__ off_tap, unsigned pos, T offv[ND]) {
#pragma unroll
    for (int a = 0; a < ND; ++a) offv[a] = off_tap[(size_t)a * P.outV + pos];
}

template <typename T, int ND>
__device__ inline void tap_setup(const Params& P, const T offv[ND], const int ib[ND], const int kd[ND],
                                 TapGeo<T, ND>& t);

// convenience form: `off_tap` points at offset[n][dg][tap][0][0]
template <typename T, int ND>
__device__ inline void tap_setup(const Params& P, const T* __restrict__ off_tap, unsigned pos,
                                 const int ib[ND], const int kd[ND], TapGeo<T, ND>& t) {
    T offv[ND];
    load_offsets<T, ND>(P, off_tap, pos, offv);
    tap_setup<T, ND>(P, offv, ib, kd, t);
}

template <typename T, int ND>
__device__ inline void tap_setup(const Params& P, const T offv[ND], const int ib[ND], const int kd[ND],
                                 TapGeo<T, ND>& t) {
    bool inside = true;
    int lo[ND], hi[ND];
#pragma unroll
    for (int a = 0; a < ND; ++a) {
        const int size = P.in[slot<ND>(a)];
        // integer part formed in int and converted once, then the offset is added (reference:
        // `l_in + l_kernel*dilation_l + data_offset_base_ptr[...]`)
        const T p = (T)(ib[a] + kd[a]) + offv[a];
        t.p[a] = p;
        inside = inside && (p > (T)-1) && (p < (T)size);
        const int l = (int)p;                                   // truncation toward zero
        lo[a] = l;
        hi[a] = (p >= (T)(size - 1) || p <= (T)0) ? l : l + 1;  // rim: high corner collapses
        t.f[a] = p - (T)l;
    }
    t.inside = inside;
#pragma unroll
    for (int a = 0; a < ND; ++a) { t.lo[a] = lo[a]; t.hi[a] = hi[a]; }
    if constexpr (ND == 3) {
        const unsigned s1 = P.in[2], s2 = P.in[1] * P.in[2];
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const int l = (c & 4) ? hi[0] : lo[0], h = (c & 2) ? hi[1] : lo[1], w = (c & 1) ? hi[2] : lo[2];
            t.idx[c] = inside ? (unsigned)l * s2 + (unsigned)h * s1 + (unsigned)w : 0u;
        }
    } else {
        const unsigned s1 = P.in[2];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int h = (c & 2) ? hi[0] : lo[0], w = (c & 1) ? hi[1] : lo[1];
            t.idx[c] = inside ? (unsigned)h * s1 + (unsigned)w : 0u;
        }
    }
}

// The same without corner indices (t.idx stays unset): for callers that sample from an LDS halo
// and need global offsets only for the rare samples that reach past it (tap_corner_idx).
template <typename T, int ND>
__device__ inline void tap_setup_noidx(const Params& P, const T offv[ND], const int ib[ND], const int kd[ND],
                                       TapGeo<T, ND>& t) {
    bool inside = true;
#pragma unroll
    for (int a = 0; a < ND; ++a) {
        const int size = P.in[slot<ND>(a)];
        const T p = (T)(ib[a] + kd[a]) + offv[a];
        t.p[a] = p;
        inside = inside && (p > (T)-1) && (p < (T)size);
        const int l = (int)p;
        t.lo[a] = l;
        t.hi[a] = (p >= (T)(size - 1) || p <= (T)0) ? l : l + 1;
        t.f[a] = p - (T)l;
    }
    t.inside = inside;
}
// Corner offsets in units of `unit` (voxel index * unit), all zero unless `ok`: the low corner's
// offset from three integer multiplies, the other corners by adding the strides of the axes whose
// high corner has not collapsed onto the low one (a multiply per corner costs four times an add).
template <typename T, int ND>
__device__ inline void tap_corner_offsets(const Params& P, const TapGeo<T, ND>& t, bool ok, unsigned unit,
                                          unsigned o[1 << ND]) {
    if constexpr (ND == 3) {
        const unsigned u2 = unit, u1 = (unsigned)P.in[2] * unit, u0 = (unsigned)P.in[1] * u1;       // uniform
        const unsigned base = (((unsigned)t.lo[0] * (unsigned)P.in[1] + (unsigned)t.lo[1]) * (unsigned)P.in[2] + (unsigned)t.lo[2]) * unit;
        const unsigned b = ok ? base : 0u;
        const unsigned s0 = (ok && t.hi[0] != t.lo[0]) ? u0 : 0u, s1 = (ok && t.hi[1] != t.lo[1]) ? u1 : 0u;
        const unsigned s2 = (ok && t.hi[2] != t.lo[2]) ? u2 : 0u;
        o[0] = b;      o[1] = b + s2;      o[2] = b + s1;      o[3] = b + s1 + s2;
        o[4] = b + s0; o[5] = b + s0 + s2; o[6] = b + s0 + s1; o[7] = b + s0 + s1 + s2;
    } else {
        const unsigned u1 = unit, u0 = (unsigned)P.in[2] * unit;
        const unsigned base = ((unsigned)t.lo[0] * (unsigned)P.in[2] + (unsigned)t.lo[1]) * unit;
        const unsigned b = ok ? base : 0u;
        const unsigned s0 = (ok && t.hi[0] != t.lo[0]) ? u0 : 0u, s1 = (ok && t.hi[1] != t.lo[1]) ? u1 : 0u;
        o[0] = b; o[1] = b + s1; o[2] = b + s0; o[3] = b + s0 + s1;
    }
}

template <typename T, int ND>
__device__ inline void tap_corner_idx(const Params& P, TapGeo<T, ND>& t) {
    if constexpr (ND == 3) {
        const unsigned s1 = P.in[2], s2 = P.in[1] * P.in[2];
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const int l = (c & 4) ? t.hi[0] : t.lo[0], h = (c & 2) ? t.hi[1] : t.lo[1], w = (c & 1) ? t.hi[2] : t.lo[2];
            t.idx[c] = t.inside ? (unsigned)l * s2 + (unsigned)h * s1 + (unsigned)w : 0u;
        }
    } else {
        const unsigned s1 = P.in[2];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int h = (c & 2) ? t.hi[0] : t.lo[0], w = (c & 1) ? t.hi[1] : t.lo[1];
            t.idx[c] = t.inside ? (unsigned)h * s1 + (unsigned)w : 0u;
        }
    }
}

// Interpolated value of one channel: lerp along w, then h, then l (reference order,
// deform3d kernel.cu:48-56, deform2d_double kernel.cu:50-53).  `chan` points at the channel's
// first voxel; `voff` are the corner offsets (possibly biased by the caller, see kernels).
// Split into the loads and the arithmetic so that callers can keep the loads of the next step in
// flight while the current one is interpolated.
template <typename T, int ND>
__device__ inline void load_corners(const T* __restrict__ chan, const unsigned* voff, T c[1 << ND]) {
#pragma unroll
    for (int i = 0; i < (1 << ND); ++i) c[i] = chan[voff[i]];
}

template <typename T, int ND>
__device__ inline T interp(const T c[1 << ND], const T* f) {
    if constexpr (ND == 3) {
        const T fw = f[2], gw = (T)1 - fw, fh = f[1], gh = (T)1 - fh, fl = f[0], gl = (T)1 - fl;
        const T c00 = c[0] * gw + c[1] * fw, c01 = c[2] * gw + c[3] * fw;
        const T c10 = c[4] * gw + c[5] * fw, c11 = c[6] * gw + c[7] * fw;
        const T c0 = c00 * gh + c01 * fh, c1 = c10 * gh + c11 * fh;
        return c0 * gl + c1 * fl;
    } else {
        const T fw = f[1], gw = (T)1 - fw, fh = f[0], gh = (T)1 - fh;
        const T c0 = c[0] * gw + c[1] * fw, c1 = c[2] * gw + c[3] * fw;
        return c0 * gh + c1 * fh;
    }
}

template <typename T, int ND>
__device__ inline T sample(const T* __restrict__ chan, const unsigned* voff, const T* f) {
    T c[1 << ND];
    load_corners<T, ND>(chan, voff, c);
    return interp<T, ND>(c, f);
}

__device__ inline void atomic_add(float* p, float v) { unsafeAtomicAdd(p, v); }
__device__ inline void atomic_add(double* p, double v) { unsafeAtomicAdd(p, v); }
// LDS float add without return value (ds_add_f32 / ds_add_f64)
template <typename T> __device__ inline void lds_atomic_add(T* p, T v) {
    (void)__hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

}  // namespace dcn
