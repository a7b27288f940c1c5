// CPU oracle for the deformable-convolution hot path.  TEST INFRASTRUCTURE ONLY.
//
// This file restates, for the host CPU, the algorithm of lshiwjx/deform_conv3d_pytorch_op:
// deformable im2col into a per-sample column buffer, one GEMM per convolution group, col2im
// scatter for grad-input, col2im_coord for grad-offset and a second im2col + GEMM for
// grad-weight.  It exists so that the HIP library can be checked against the reference's
// arithmetic and so that a CPU baseline can be timed next to the GPU numbers.  Nothing in the
// shipped package may call it: only tests, the smoke check and the benchmark's cpu_baseline leg.
//
// Reference files each part follows (paths relative to the reference checkout):
//   sampler 3-D            deform3d/lib/deform_conv3d_cuda_kernel.cu:12-59
//   sampler 2-D            deform2d_double/lib/deform_conv2d_cuda_kernel.cu:25-56
//                          (deform2d/lib/deform_conv2d_cuda_kernel.cu:12-43 is its float twin)
//   im2col 3-D / 2-D       deform3d/...kernel.cu:72-130 ; deform2d_double/...kernel.cu:69-123
//   col2im_input 3-D / 2-D deform3d/...kernel.cu:185-297 ; deform2d_double/...kernel.cu:166-240
//   col2im_offset 3-D      deform3d/...kernel.cu:352-484 (with the out-of-range branches :470-481)
//   col2im_offset 2-D      deform2d_double/...kernel.cu:282-367 (no out-of-range branch)
//   sequencing + GEMMs     deform3d/lib/deform_conv3d_cuda.cpp:105-158, 186-253, 278-330
//                          deform2d_double/lib/deform_conv2d_cuda.cpp:97-148, 176-239, 265-318
//   output size            deform3d/lib/deform_conv3d_cuda.cpp:15-17
//
// Parity status.  The reference holds no golden vectors, so every function here is pinned by
// independent checks in tests/ (grid_sample composite, F.conv for zero offsets, brute force,
// adjoint identity, hand cases).  One part has no independent pin: the 3-D out-of-range
// grad-offset branches (:470-481) are not the derivative of anything; they are restated
// literally, including the comparison against the *length* extent on the h and w axes, and are
// "parity unpinned" beyond hand-built closed-form cases.
//
// The GEMMs are cuBLAS Sgemm/Dgemm in the reference (PyTorch 0.3.0 THC, un-vendored); only the
// summation order is unspecified there.  `acc64 != 0` accumulates dot products in double even
// for float data (closest to the exact sum, used by tests); `acc64 == 0` accumulates in the
// data type (what Sgemm does, used for the timed CPU baseline).
//
// Build: see oracle/Makefile (g++ -O2 -fopenmp -ffp-contract=off).

#include <cstdint>
#include <cstring>
#include <cstdlib>
#include <vector>

namespace {

struct Geom {
    int nd;                 // 2 or 3
    int N, C_in, C_out;
    int in[3];              // l, h, w  (l == 1 for 2-D)
    int out[3];
    int k[3], pad[3], stride[3], dil[3];
    int cpg;                // channels per deformable group
    int groups;             // convolution groups
    long inV() const { return (long)in[0] * in[1] * in[2]; }
    long outV() const { return (long)out[0] * out[1] * out[2]; }
    int kV() const { return k[0] * k[1] * k[2]; }
    int DG() const { return C_in / cpg; }
};

// geometry array layout shared with oracle/dcn_oracle.py
Geom unpack(const int* g) {
    Geom G;
    G.nd = g[0]; G.N = g[1]; G.C_in = g[2]; G.C_out = g[3];
    for (int a = 0; a < 3; ++a) {
        G.in[a] = g[4 + a]; G.out[a] = g[7 + a]; G.k[a] = g[10 + a];
        G.pad[a] = g[13 + a]; G.stride[a] = g[16 + a]; G.dil[a] = g[19 + a];
    }
    G.cpg = g[22]; G.groups = g[23];
    return G;
}

// ---------------------------------------------------------------------------------------------
// Sampling geometry of one (tap, position): the real coordinate per axis, the inside test and
// the corner indices / fractions.  3-D: deform3d kernel.cu:21-26,40-45 ; 2-D: deform2d_double
// kernel.cu:31-34,43-46.  `int(p)` truncates toward zero; the high corner collapses onto the low
// one when p <= 0 or p >= size-1, so the one-voxel rim replicates the edge.
template <typename T>
struct Tap3 {
    T p[3];
    bool inside;
    int lo[3], hi[3];
    T f[3];     // "l_*" in the reference: p - lo
    T g[3];     // "h_*" in the reference: 1 - f
};

template <typename T>
inline void corners(T p, int size, int& lo, int& hi, T& f, T& g) {
    lo = (int)p;
    hi = (p >= size - 1 || p <= 0) ? lo : lo + 1;
    f = p - lo;
    g = 1 - f;
}

template <typename T>
inline Tap3<T> make_tap(const Geom& G, const T* off_n, int dg, int tap, const int kk[3], const int o[3]) {
    Tap3<T> t;
    const long outV = G.outV();
    const long pos = ((long)o[0] * G.out[1] + o[1]) * G.out[2] + o[2];
    const T* base = off_n + ((long)dg * G.kV() + tap) * G.nd * outV;
    t.inside = true;
    for (int a = 0; a < 3; ++a) {
        const int ax = a - (3 - G.nd);       // axis index inside the offset tensor, <0: absent
        const int ip = o[a] * G.stride[a] - G.pad[a] + kk[a] * G.dil[a];
        // reference: `l_in + l_kernel*dilation_l + data_offset[...]` -> int sum converted once.
        T p = (T)ip;
        if (ax >= 0) p = p + base[ax * outV + pos];
        t.p[a] = p;
        if (!(p > -1 && p < G.in[a])) t.inside = false;
    }
    if (t.inside)
        for (int a = 0; a < 3; ++a) corners<T>(t.p[a], G.in[a], t.lo[a], t.hi[a], t.f[a], t.g[a]);
    return t;
}

// Tri_Linear (deform3d kernel.cu:29-56): lerp along w, then h, then l.
template <typename T>
inline T sample3(const T* im, const Geom& G, const Tap3<T>& t) {
    const long s1 = G.in[2], s2 = (long)G.in[1] * G.in[2];
    const T c000 = im[t.lo[0] * s2 + t.lo[1] * s1 + t.lo[2]];
    const T c001 = im[t.lo[0] * s2 + t.lo[1] * s1 + t.hi[2]];
    const T c010 = im[t.lo[0] * s2 + t.hi[1] * s1 + t.lo[2]];
    const T c011 = im[t.lo[0] * s2 + t.hi[1] * s1 + t.hi[2]];
    const T c100 = im[t.hi[0] * s2 + t.lo[1] * s1 + t.lo[2]];
    const T c101 = im[t.hi[0] * s2 + t.lo[1] * s1 + t.hi[2]];
    const T c110 = im[t.hi[0] * s2 + t.hi[1] * s1 + t.lo[2]];
    const T c111 = im[t.hi[0] * s2 + t.hi[1] * s1 + t.hi[2]];
    const T c00 = c000 * t.g[2] + c001 * t.f[2];
    const T c01 = c010 * t.g[2] + c011 * t.f[2];
    const T c10 = c100 * t.g[2] + c101 * t.f[2];
    const T c11 = c110 * t.g[2] + c111 * t.f[2];
    const T c0 = c00 * t.g[1] + c01 * t.f[1];
    const T c1 = c10 * t.g[1] + c11 * t.f[1];
    return c0 * t.g[0] + c1 * t.f[0];
}

// Bi_Linear (deform2d_double kernel.cu:37-53).  Axis 0 is the dummy length axis (size 1).
template <typename T>
inline T sample2(const T* im, const Geom& G, const Tap3<T>& t) {
    const long s1 = G.in[2];
    const T c00 = im[t.lo[1] * s1 + t.lo[2]];
    const T c01 = im[t.lo[1] * s1 + t.hi[2]];
    const T c10 = im[t.hi[1] * s1 + t.lo[2]];
    const T c11 = im[t.hi[1] * s1 + t.hi[2]];
    const T c0 = c00 * t.g[2] + c01 * t.f[2];
    const T c1 = c10 * t.g[2] + c11 * t.f[2];
    return c0 * t.g[1] + c1 * t.f[1];
}

inline void tap_to_k(const Geom& G, int tap, int kk[3]) {
    kk[2] = tap % G.k[2];
    kk[1] = tap / G.k[2] % G.k[1];
    kk[0] = tap / G.k[2] / G.k[1];
}

// ---------------------------------------------------------------------------------------------
// Deformable im2col of one sample: col[(c*kV + tap), pos].
template <typename T>
void im2col(const Geom& G, const T* im_n, const T* off_n, T* col) {
    const long outV = G.outV(), inV = G.inV();
    const int kV = G.kV();
#pragma omp parallel for collapse(2) schedule(static)
    for (int c = 0; c < G.C_in; ++c)
        for (int tap = 0; tap < kV; ++tap) {
            int kk[3]; tap_to_k(G, tap, kk);
            const int dg = c / G.cpg;
            const T* im = im_n + c * inV;
            T* row = col + ((long)c * kV + tap) * outV;
            int o[3];
            for (o[0] = 0; o[0] < G.out[0]; ++o[0])
                for (o[1] = 0; o[1] < G.out[1]; ++o[1])
                    for (o[2] = 0; o[2] < G.out[2]; ++o[2]) {
                        const Tap3<T> t = make_tap<T>(G, off_n, dg, tap, kk, o);
                        T v = 0;
                        if (t.inside) v = (G.nd == 3) ? sample3<T>(im, G, t) : sample2<T>(im, G, t);
                        row[((long)o[0] * G.out[1] + o[1]) * G.out[2] + o[2]] = v;
                    }
        }
}

// col2im for grad-input of one sample (accumulates into gim_n, caller zero-fills).  Products are
// formed as (w_l*w_h*w_w)*gcol like the reference's atomicAdd arguments (3-D :264-295, 2-D
// :223-238).  Channels are independent, so parallelising over c needs no atomics.
template <typename T>
void col2im_input(const Geom& G, const T* col, const T* off_n, T* gim_n) {
    const long outV = G.outV(), inV = G.inV();
    const int kV = G.kV();
    const long s1 = G.in[2], s2 = (long)G.in[1] * G.in[2];
#pragma omp parallel for schedule(static)
    for (int c = 0; c < G.C_in; ++c) {
        const int dg = c / G.cpg;
        T* gim = gim_n + c * inV;
        int o[3];
        for (o[0] = 0; o[0] < G.out[0]; ++o[0])
            for (o[1] = 0; o[1] < G.out[1]; ++o[1])
                for (o[2] = 0; o[2] < G.out[2]; ++o[2]) {
                    const long pos = ((long)o[0] * G.out[1] + o[1]) * G.out[2] + o[2];
                    for (int tap = 0; tap < kV; ++tap) {
                        int kk[3]; tap_to_k(G, tap, kk);
                        const Tap3<T> t = make_tap<T>(G, off_n, dg, tap, kk, o);
                        if (!t.inside) continue;
                        const T gc = col[((long)c * kV + tap) * outV + pos];
                        if (G.nd == 3) {
                            gim[t.lo[0] * s2 + t.lo[1] * s1 + t.lo[2]] += t.g[0] * t.g[1] * t.g[2] * gc;
                            gim[t.lo[0] * s2 + t.lo[1] * s1 + t.hi[2]] += t.g[0] * t.g[1] * t.f[2] * gc;
                            gim[t.lo[0] * s2 + t.hi[1] * s1 + t.lo[2]] += t.g[0] * t.f[1] * t.g[2] * gc;
                            gim[t.lo[0] * s2 + t.hi[1] * s1 + t.hi[2]] += t.g[0] * t.f[1] * t.f[2] * gc;
                            gim[t.hi[0] * s2 + t.lo[1] * s1 + t.lo[2]] += t.f[0] * t.g[1] * t.g[2] * gc;
                            gim[t.hi[0] * s2 + t.lo[1] * s1 + t.hi[2]] += t.f[0] * t.g[1] * t.f[2] * gc;
                            gim[t.hi[0] * s2 + t.hi[1] * s1 + t.lo[2]] += t.f[0] * t.f[1] * t.g[2] * gc;
                            gim[t.hi[0] * s2 + t.hi[1] * s1 + t.hi[2]] += t.f[0] * t.f[1] * t.f[2] * gc;
                        } else {
                            gim[t.lo[1] * s1 + t.lo[2]] += t.g[1] * t.g[2] * gc;
                            gim[t.lo[1] * s1 + t.hi[2]] += t.g[1] * t.f[2] * gc;
                            gim[t.hi[1] * s1 + t.lo[2]] += t.f[1] * t.g[2] * gc;
                            gim[t.hi[1] * s1 + t.hi[2]] += t.f[1] * t.f[2] * gc;
                        }
                    }
                }
    }
}

// col2im_coord for grad-offset of one sample (plain store, every element written).
template <typename T>
void col2im_offset(const Geom& G, const T* col, const T* im_n, const T* off_n, T* goff_n) {
    const long outV = G.outV(), inV = G.inV();
    const int kV = G.kV(), DG = G.DG(), nd = G.nd;
    const long s1 = G.in[2], s2 = (long)G.in[1] * G.in[2];
#pragma omp parallel for collapse(2) schedule(static)
    for (int dg = 0; dg < DG; ++dg)
        for (int tap = 0; tap < kV; ++tap) {
            int kk[3]; tap_to_k(G, tap, kk);
            int o[3];
            for (o[0] = 0; o[0] < G.out[0]; ++o[0])
                for (o[1] = 0; o[1] < G.out[1]; ++o[1])
                    for (o[2] = 0; o[2] < G.out[2]; ++o[2]) {
                        const long pos = ((long)o[0] * G.out[1] + o[1]) * G.out[2] + o[2];
                        const Tap3<T> t = make_tap<T>(G, off_n, dg, tap, kk, o);
                        for (int ax = 0; ax < nd; ++ax) {
                            T val = 0;
                            for (int i = 0; i < G.cpg; ++i) {
                                const int c = dg * G.cpg + i;
                                const T gc = col[((long)c * kV + tap) * outV + pos];
                                const T* im = im_n + c * inV;
                                if (t.inside) {
                                    if (nd == 3) {
                                        const T c000 = im[t.lo[0] * s2 + t.lo[1] * s1 + t.lo[2]];
                                        const T c001 = im[t.lo[0] * s2 + t.lo[1] * s1 + t.hi[2]];
                                        const T c010 = im[t.lo[0] * s2 + t.hi[1] * s1 + t.lo[2]];
                                        const T c011 = im[t.lo[0] * s2 + t.hi[1] * s1 + t.hi[2]];
                                        const T c100 = im[t.hi[0] * s2 + t.lo[1] * s1 + t.lo[2]];
                                        const T c101 = im[t.hi[0] * s2 + t.lo[1] * s1 + t.hi[2]];
                                        const T c110 = im[t.hi[0] * s2 + t.hi[1] * s1 + t.lo[2]];
                                        const T c111 = im[t.hi[0] * s2 + t.hi[1] * s1 + t.hi[2]];
                                        const T fl = t.f[0], gl = t.g[0], fh = t.f[1], gh = t.g[1],
                                                fw = t.f[2], gw = t.g[2];
                                        if (ax == 0)        // :446-450
                                            val += gc * (c100 * gh * gw + c101 * gh * fw +
                                                         c110 * fh * gw + c111 * fh * fw -
                                                         c000 * gh * gw - c001 * gh * fw -
                                                         c010 * fh * gw - c011 * fh * fw);
                                        else if (ax == 1)   // :453-457
                                            val += gc * (c010 * gl * gw + c011 * gl * fw +
                                                         c110 * fl * gw + c111 * fl * fw -
                                                         c000 * gl * gw - c001 * gl * fw -
                                                         c100 * fl * gw - c101 * fl * fw);
                                        else                // :460-464
                                            val += gc * (c001 * gh * gl + c101 * gh * fl +
                                                         c011 * fh * gl + c111 * fh * fl -
                                                         c000 * gh * gl - c100 * gh * fl -
                                                         c010 * fh * gl - c110 * fh * fl);
                                    } else {
                                        const T c00 = im[t.lo[1] * s1 + t.lo[2]];
                                        const T c01 = im[t.lo[1] * s1 + t.hi[2]];
                                        const T c10 = im[t.hi[1] * s1 + t.lo[2]];
                                        const T c11 = im[t.hi[1] * s1 + t.hi[2]];
                                        const T fh = t.f[1], gh = t.g[1], fw = t.f[2], gw = t.g[2];
                                        if (ax == 0)        // deform2d_double :352-354
                                            val += gc * (c11 * fw + c10 * gw - c01 * fw - c00 * gw);
                                        else                // :357-359
                                            val += gc * (c01 * gh + c11 * fh - c00 * gh - c10 * fh);
                                    }
                                } else if (nd == 3) {
                                    // deform3d :470-481 -- "pull back" heuristic for samples that
                                    // left the volume.  All three upper tests compare against the
                                    // LENGTH extent (in[0]); that is what the reference does.
                                    const T a = gc > 0 ? gc : -gc;
                                    if (t.p[0] <= -1 && ax == 0) val += -a;
                                    else if (t.p[0] >= G.in[0] && ax == 0) val += a;
                                    else if (t.p[1] <= -1 && ax == 1) val += -a;
                                    else if (t.p[1] >= G.in[0] && ax == 1) val += a;
                                    else if (t.p[2] <= -1 && ax == 2) val += -a;
                                    else if (t.p[2] >= G.in[0] && ax == 2) val += a;
                                }
                            }
                            goff_n[(((long)dg * kV + tap) * nd + ax) * outV + pos] = val;
                        }
                    }
        }
}

// ---------------------------------------------------------------------------------------------
// The three GEMMs (row-major views), one call per sample and convolution group.
// G1: out[M,P]  = W[M,K] * col[K,P]            (deform3d cpp:140-148, beta 0)
// G2: col[K,P]  = W[M,K]^T * gout[M,P]         (deform3d cpp:213-220, beta 0)
// G3: gW[M,K]  += gout[M,P] * col[K,P]^T       (deform3d cpp:314-320, beta 1)
template <typename T, typename A>
void gemm_nn(int M, int K, long P, const T* W, const T* col, T* out) {
#pragma omp parallel
    {
        std::vector<A> acc(P);
#pragma omp for schedule(static)
        for (int m = 0; m < M; ++m) {
            for (long p = 0; p < P; ++p) acc[p] = 0;
            for (int k = 0; k < K; ++k) {
                const A a = (A)W[(long)m * K + k];
                const T* cr = col + (long)k * P;
#pragma omp simd
                for (long p = 0; p < P; ++p) acc[p] += a * (A)cr[p];
            }
            for (long p = 0; p < P; ++p) out[(long)m * P + p] = (T)acc[p];
        }
    }
}

template <typename T, typename A>
void gemm_tn(int M, int K, long P, const T* W, const T* gout, T* col) {
#pragma omp parallel
    {
        std::vector<A> acc(P);
#pragma omp for schedule(static)
        for (int k = 0; k < K; ++k) {
            for (long p = 0; p < P; ++p) acc[p] = 0;
            for (int m = 0; m < M; ++m) {
                const A a = (A)W[(long)m * K + k];
                const T* gr = gout + (long)m * P;
#pragma omp simd
                for (long p = 0; p < P; ++p) acc[p] += a * (A)gr[p];
            }
            for (long p = 0; p < P; ++p) col[(long)k * P + p] = (T)acc[p];
        }
    }
}

template <typename T, typename A>
void gemm_nt_acc(int M, int K, long P, const T* gout, const T* col, T* gW) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int m = 0; m < M; ++m)
        for (int k = 0; k < K; ++k) {
            const T* gr = gout + (long)m * P;
            const T* cr = col + (long)k * P;
            A s = 0;
#pragma omp simd reduction(+ : s)
            for (long p = 0; p < P; ++p) s += (A)gr[p] * (A)cr[p];
            gW[(long)m * K + k] += (T)s;
        }
}

// ---------------------------------------------------------------------------------------------
// Host sequencing: serial loop over samples, column buffer reused, one GEMM per group.
template <typename T, typename A>
void forward(const Geom& G, const T* in, const T* w, const T* off, T* out, T* col) {
    const long inV = G.inV(), outV = G.outV();
    const int kV = G.kV(), M = G.C_out / G.groups, K = G.C_in / G.groups * kV;
    const long offC = (long)G.DG() * kV * G.nd;
    for (int n = 0; n < G.N; ++n) {
        im2col<T>(G, in + (long)n * G.C_in * inV, off + n * offC * outV, col);
        for (int g = 0; g < G.groups; ++g)
            gemm_nn<T, A>(M, K, outV, w + (long)g * M * K, col + (long)g * K * outV,
                          out + ((long)n * G.C_out + (long)g * M) * outV);
    }
}

template <typename T, typename A>
void backward_input_offset(const Geom& G, const T* in, const T* w, const T* off, const T* gout,
                           T* gin, T* goff, T* col) {
    const long inV = G.inV(), outV = G.outV();
    const int kV = G.kV(), M = G.C_out / G.groups, K = G.C_in / G.groups * kV;
    const long offC = (long)G.DG() * kV * G.nd;
    for (int n = 0; n < G.N; ++n) {
        for (int g = 0; g < G.groups; ++g)
            gemm_tn<T, A>(M, K, outV, w + (long)g * M * K,
                          gout + ((long)n * G.C_out + (long)g * M) * outV, col + (long)g * K * outV);
        col2im_offset<T>(G, col, in + (long)n * G.C_in * inV, off + n * offC * outV,
                         goff + n * offC * outV);
        col2im_input<T>(G, col, off + n * offC * outV, gin + (long)n * G.C_in * inV);
    }
}

template <typename T, typename A>
void backward_weight(const Geom& G, const T* in, const T* off, const T* gout, T* gw, T* col) {
    const long inV = G.inV(), outV = G.outV();
    const int kV = G.kV(), M = G.C_out / G.groups, K = G.C_in / G.groups * kV;
    const long offC = (long)G.DG() * kV * G.nd;
    for (int n = 0; n < G.N; ++n) {
        im2col<T>(G, in + (long)n * G.C_in * inV, off + n * offC * outV, col);
        for (int g = 0; g < G.groups; ++g)
            gemm_nt_acc<T, A>(M, K, outV, gout + ((long)n * G.C_out + (long)g * M) * outV,
                              col + (long)g * K * outV, gw + (long)g * M * K);
    }
}

}  // namespace

// ---------------------------------------------------------------------------------------------
// C ABI (host pointers).  dtype: 0 = float, 1 = double.  `geom` is the 24-int array described in
// unpack().  `columns` is the caller's [C_in*kV, outV] workspace, as in the reference.
// All return 0; shape validation lives in the Python wrapper.
extern "C" {

int dcn_oracle_output_size(int in, int pad, int k, int stride) {
    // deform3d/lib/deform_conv3d_cuda.cpp:15-17 -- dilation is not part of the formula.
    return (in + 2 * pad - k) / stride + 1;
}

#define DISPATCH(CALL_F32A32, CALL_F32A64, CALL_F64)      \
    if (dtype == 0) { if (acc64) { CALL_F32A64; } else { CALL_F32A32; } } \
    else { CALL_F64; }

int dcn_oracle_forward(int dtype, int acc64, const int* geom, const void* in, const void* w,
                       const void* off, void* out, void* col) {
    const Geom G = unpack(geom);
    DISPATCH((forward<float, float>(G, (const float*)in, (const float*)w, (const float*)off, (float*)out, (float*)col)),
             (forward<float, double>(G, (const float*)in, (const float*)w, (const float*)off, (float*)out, (float*)col)),
             (forward<double, double>(G, (const double*)in, (const double*)w, (const double*)off, (double*)out, (double*)col)));
    return 0;
}

int dcn_oracle_backward_input_offset(int dtype, int acc64, const int* geom, const void* in,
                                     const void* w, const void* off, const void* gout, void* gin,
                                     void* goff, void* col) {
    const Geom G = unpack(geom);
    DISPATCH((backward_input_offset<float, float>(G, (const float*)in, (const float*)w, (const float*)off, (const float*)gout, (float*)gin, (float*)goff, (float*)col)),
             (backward_input_offset<float, double>(G, (const float*)in, (const float*)w, (const float*)off, (const float*)gout, (float*)gin, (float*)goff, (float*)col)),
             (backward_input_offset<double, double>(G, (const double*)in, (const double*)w, (const double*)off, (const double*)gout, (double*)gin, (double*)goff, (double*)col)));
    return 0;
}

int dcn_oracle_backward_weight(int dtype, int acc64, const int* geom, const void* in,
                               const void* off, const void* gout, void* gw, void* col) {
    const Geom G = unpack(geom);
    DISPATCH((backward_weight<float, float>(G, (const float*)in, (const float*)off, (const float*)gout, (float*)gw, (float*)col)),
             (backward_weight<float, double>(G, (const float*)in, (const float*)off, (const float*)gout, (float*)gw, (float*)col)),
             (backward_weight<double, double>(G, (const double*)in, (const double*)off, (const double*)gout, (double*)gw, (double*)col)));
    return 0;
}

// Single stages on one sample, for pinning each part separately.
int dcn_oracle_im2col(int dtype, const int* geom, const void* im_n, const void* off_n, void* col) {
    const Geom G = unpack(geom);
    if (dtype == 0) im2col<float>(G, (const float*)im_n, (const float*)off_n, (float*)col);
    else im2col<double>(G, (const double*)im_n, (const double*)off_n, (double*)col);
    return 0;
}

int dcn_oracle_col2im_input(int dtype, const int* geom, const void* col, const void* off_n, void* gim_n) {
    const Geom G = unpack(geom);
    if (dtype == 0) col2im_input<float>(G, (const float*)col, (const float*)off_n, (float*)gim_n);
    else col2im_input<double>(G, (const double*)col, (const double*)off_n, (double*)gim_n);
    return 0;
}

int dcn_oracle_col2im_offset(int dtype, const int* geom, const void* col, const void* im_n,
                             const void* off_n, void* goff_n) {
    const Geom G = unpack(geom);
    if (dtype == 0) col2im_offset<float>(G, (const float*)col, (const float*)im_n, (const float*)off_n, (float*)goff_n);
    else col2im_offset<double>(G, (const double*)col, (const double*)im_n, (const double*)off_n, (double*)goff_n);
    return 0;
}

}  // extern "C"
