// Forward kernel with the input halo in LDS, four channels of a voxel side by side.
//
//   out[n][g*M + m][pos] = sum_{cl,tap} W[g*M+m][cl][tap] * sample(in[n][g*Cg+cl], tap, pos)  (+ bias)
//
// replaces deformable_im2col + the per-group Sgemm of the reference
// (deform3d/lib/deform_conv3d_cuda.cpp:110-148, deform2d_double/lib/deform_conv2d_cuda.cpp:102-138).
//
// Lane roles.  A wavefront owns TN output positions; lane (j, q) works on position j and on
// reduction slot q of the MFMA (B[k = q][col = j]).  The KL reduction slots of one MFMA step are KL
// consecutive TAPS of one channel: lane group q samples tap tg*KL + q, so every lane derives the
// geometry of ONE (tap, position) per tap group and no two lanes of a wavefront repeat each other's
// work.  The sample then serves four channels at a time: the halo holds the four channels of a
// voxel in 16 (32) consecutive bytes, one wide LDS read per corner fetches all of them, and the
// interpolated values of the four channels are the B operands of four MFMA steps.
#pragma once
#include <limits>
#include "dcn_kernels.h"

#include <type_traits>

namespace dcn {

constexpr int FQ = 4;              // channels per group: one wide LDS read per corner

// Weights of the forward kernel: one slab per group of four channels (groups start at the first
// channel of a segment -- the channels shared by one deformable group and one convolution group --
// and every fourth after it), in the order the lanes consume them:
//   Wq[slab][tap group][row tile][q][j][e] = W[m = tile*TN + j][channel = first + e][tap = tg*KL + q]
// zero past M, past the last tap and past the segment.  A lane's four values of one (tap group, row
// tile) are 16 (32) contiguous bytes and a wavefront's are one contiguous run.
template <typename T>
__host__ __device__ inline size_t forward_slab_elems(int kV, int Mp) {
    return (size_t)((kV + Mma<T>::KL - 1) / Mma<T>::KL) * Mp * Mma<T>::KL * FQ;
}

// With pc.sel set the launch has one block more, which chooses the halo plan from the offsets.
template <typename T, typename S = T>
__global__ void pack_forward_weight_kernel(Params P, const S* __restrict__ W, S* __restrict__ Wq, PlanChoice pc,
                                           const S* __restrict__ off, size_t n_off) {
    using MM = Mma<T>;
    constexpr int TN = MM::TN, KL = MM::KL;
    const unsigned pack_blocks = pc.sel ? gridDim.x - 1 : gridDim.x;
    if (blockIdx.x == pack_blocks) {
        choose_plan(pc, off, n_off);
        return;
    }
    const int mtiles = P.Mp / TN;
    const size_t per_slab = forward_slab_elems<T>(P.kV, P.Mp);
    const size_t total = (size_t)chunk_candidates<FQ>(P.cpg, P.Cg, P.C_in) * per_slab;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)pack_blocks * blockDim.x) {
        const int c0 = chunk_candidate<FQ>(P.cpg, P.Cg, (int)(i / per_slab));       // candidate first channel of a group
        const int seg_b = max(c0 / P.cpg * P.cpg, c0 / P.Cg * P.Cg);
        if ((c0 - seg_b) % FQ) continue;
        const int seg_e = min((c0 / P.cpg + 1) * P.cpg, (c0 / P.Cg + 1) * P.Cg);
        size_t r = i % per_slab;
        const int e = (int)(r % FQ); r /= FQ;
        const int j = (int)(r % TN); r /= TN;
        const int q = (int)(r % KL); r /= KL;
        const int tile = (int)(r % mtiles);
        const int tg = (int)(r / mtiles);
        const int m = tile * TN + j, tap = tg * KL + q, c = c0 + e, g = c0 / P.Cg;
        S v = S();
        if (m < P.M && tap < P.kV && c < seg_e) v = W[(((size_t)g * P.M + m) * P.Cg + (c - g * P.Cg)) * P.kV + tap];
        Wq[(size_t)chunk_slot<FQ>(P.cpg, P.Cg, c0) * per_slab + i % per_slab] = v;
    }
}

// Stage `nch` channels of the halo as groups of four: sIn[group][halo voxel][4].  Missing channels
// of a short last group and halo voxels outside the volume hold zero (a sample in the rim reads
// the latter with weight zero).
template <typename T, int WGS, typename S = T>
__device__ inline void halo_stage_quads(const Params& P, const HaloPlan& H, const S* __restrict__ chan0, int nch,
                                        const unsigned* __restrict__ sTab, T* __restrict__ sIn, int* __restrict__ nonfinite) {
    const int ngrp = (nch + FQ - 1) / FQ;
    bool bad = false;                  // a NaN or an infinity among the staged values (see halo_nonfinite)
    for (int v = threadIdx.x; v < H.hvol; v += WGS) {
        const unsigned t = sTab[v];
        const unsigned g = t == ~0u ? 0u : t;
        for (int grp = 0; grp < ngrp; ++grp) {
            T val[FQ];
#pragma unroll
            for (int e = 0; e < FQ; ++e) val[e] = Store<S>::ld(chan0[(size_t)min(grp * FQ + e, nch - 1) * P.inV + g]);
#pragma unroll
            for (int e = 0; e < FQ; ++e) bad = bad || !(fabs(val[e]) <= std::numeric_limits<T>::max());
#pragma unroll
            for (int e = 0; e < FQ; ++e)
                sIn[((size_t)grp * H.hstride + v) * FQ + e] = (grp * FQ + e < nch && t != ~0u) ? val[e] : (T)0;
        }
    }
    if (bad) *nonfinite = 1;
}

// 1-D grid of N * tiles (blocks of positions) * G * mchunks * csplit workgroups of NW wavefronts;
// dynamic LDS = cchunk * hstride * sizeof(T) + hvol * 4 with cchunk a multiple of four.
// csplit > 1: csplit workgroups share the input-channel chunks of a unit (block, group,
// output-channel chunk) -- workgroup cz takes every csplit-th -- and write partial sums without
// bias, which a second kernel adds up in a fixed order.  Two uses:
//   whole = 0 (layers with too few position blocks to fill the device): every unit is split; the
//     partial outputs are whole output tensors at part + cz * N * C_out * outV
//     (forward_join_partials_kernel);
//   whole > 0 (a grid that ends in a partly filled round of workgroups): the first `whole` units
//     run unsplit and write the output itself, the others, last in the launch, are split so that
//     the last round fills the device; their partial sums go to part as
//     [split workgroup][row of the chunk][position of the block] in launch order, i.e.
//     [unit - whole][cz] within each of the two runs of TailSplit (forward_join_tail_kernel).
// (few accumulators: four wavefronts per SIMD, i.e. at most 128 registers, also for the 512-thread
// shape, so that two of its workgroups share a CU)
// S: storage format of the tensors (see Store); T is float with a 16-bit format, and partial sums are always T.
template <typename T, int ND, int MT, int NW, typename S = T>
__global__ __launch_bounds__(NW * 64, (MT <= 2 && sizeof(T) == 4) ? 4 : 1) void forward_quad_kernel(Params P, PlanSet alts, const unsigned* __restrict__ sel,
                                                           const S* __restrict__ in,
                                                           const S* __restrict__ off, const S* __restrict__ Wq,
                                                           const S* __restrict__ bias, S* __restrict__ out,
                                                           T* __restrict__ part, int csplit, unsigned whole, TailSplit ts) {
    HaloPlan H;
    if (!chosen_halo(P, alts, sel, H)) return;          // another launch runs the chosen plan
    using MM = Mma<T>;
    constexpr int TN = MM::TN, KL = MM::KL, NC = 1 << ND, WGS = NW * 64;
    constexpr bool S16 = sizeof(S) == 2;                // 16-bit storage: 16-bit matrix instructions
    typedef T V4 __attribute__((ext_vector_type(4)));
    extern __shared__ __align__(16) unsigned char smem_raw[];
    __shared__ int sNonFinite;
    T* sIn = reinterpret_cast<T*>(smem_raw);                                            // [cchunk / 4][hstride][4]
    unsigned* sTab = reinterpret_cast<unsigned*>(sIn + (size_t)H.cchunk * H.hstride);   // [hvol]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane % TN, q = lane / TN;
    // workgroups of one tile are neighbours in an XCD-contiguous order
    unsigned wg, pslot = 0;                             // pslot: which partial sum of the split runs
    int cz = 0;
    int cch = H.cchunk;                                 // channels per LDS pass
    const bool split = csplit > 1 && blockIdx.x >= whole;
    if (!split) wg = xcd_contiguous(blockIdx.x, csplit > 1 ? whole : gridDim.x);
    else {
        const unsigned rel = blockIdx.x - whole, all = gridDim.x - whole;
        const unsigned wgsA = ts.splitB ? ts.unitsA * (unsigned)csplit : all;
        if (rel < wgsA) {
            const unsigned r = xcd_contiguous(rel, wgsA);
            wg = whole + r / (unsigned)csplit;
            cz = r % (unsigned)csplit;
            pslot = r;
        } else {
            const unsigned r = xcd_contiguous(rel - wgsA, all - wgsA);
            csplit = ts.splitB;
            wg = whole + ts.unitsA + r / (unsigned)csplit;
            cz = r % (unsigned)csplit;
            pslot = wgsA + r;
            cch = min(cch, ts.cchB);
        }
    }
    if (!split) csplit = 1;
    const unsigned gm = wg % (unsigned)(P.G * P.mchunks);
    const int g = gm / P.mchunks, mchunk = gm % P.mchunks;

    TileGeo<ND> tg_;
    tile_decode<ND>(P, H, wg / (unsigned)(P.G * P.mchunks), tg_);
    const int n = tg_.n;
    int o[ND];
    unsigned pos;
    const bool valid = tile_position<ND>(P, tg_, wave * TN + j, o, pos);
    // o * stride - pad as T: the integer part of a sampling coordinate is (T)(that + tap * dilation),
    // a sum of two small integers that is exact in T as well
    T ibf[ND];
#pragma unroll
    for (int a = 0; a < ND; ++a) ibf[a] = (T)(o[a] * P.stride[slot<ND>(a)] - P.pad[slot<ND>(a)]);
    halo_table<ND, WGS>(P, H, tg_, sTab);             // visible after the first barrier below

    typename MM::Acc acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = acc_zero<T>();

    const int ntg = (P.kV + KL - 1) / KL, mtiles = P.Mp / TN;
    const size_t per_slab = forward_slab_elems<T>(P.kV, P.Mp);
    // corner i of a sample sits at a fixed distance from its low corner (strides of the halo); a
    // corner that the reference collapses onto the low one carries weight zero instead
    unsigned coff[NC];
#pragma unroll
    for (int i = 0; i < NC; ++i)
        coff[i] = ND == 3 ? (unsigned)((((i >> 2) & 1) * H.hext[1] + ((i >> 1) & 1)) * H.hext[2] + (i & 1))
                          : (unsigned)(((i >> 1) & 1) * H.hext[2] + (i & 1));
    // this lane's weights of (tap group 0, first row tile of the chunk) inside a slab
    const unsigned w_lane = (((unsigned)mchunk * MT * KL + q) * TN + j) * FQ;
    const unsigned w_tile = (unsigned)KL * TN * FQ;               // one row tile further
    const unsigned w_tg = (unsigned)mtiles * KL * TN * FQ;        // one tap group further

    const int cg0 = g * P.Cg, cg1 = cg0 + P.Cg;
    int chunk_no = 0;
    for (int dg = cg0 / P.cpg; dg <= (cg1 - 1) / P.cpg; ++dg) {
        const int cb = max(cg0, dg * P.cpg), ce = min(cg1, (dg + 1) * P.cpg);
        const S* off_dg = off + ((size_t)n * P.DG + dg) * P.kV * ND * P.outV;
        for (int cc0 = cb; cc0 < ce; cc0 += cch) {
            if ((chunk_no++) % csplit != cz) continue;                     // another workgroup's chunk (uniform)
            const int nch = min(cch, ce - cc0);
            const int ngrp = (nch + FQ - 1) / FQ;
            const S* chan0 = in + ((size_t)n * P.C_in + cc0) * P.inV;      // workgroup-uniform
            if (threadIdx.x == 0) sNonFinite = 0;
            __syncthreads();                                               // readers of the previous chunk are done
            halo_stage_quads<T, WGS, S>(P, H, chan0, nch, sTab, sIn, &sNonFinite);
            __syncthreads();
            // Non-finite input values in this halo: the branch-free sampler reads the cell next to a
            // collapsed corner with weight 0, and 0 * inf would be NaN where the reference never
            // touches that voxel (deform3d/lib/deform_conv3d_cuda_kernel.cu:24-26).  Samples in the
            // collapse zones (p <= 0 or p >= size - 1 on some axis) then take the pass through global
            // memory, which follows the reference's corner rule.
            const bool halo_nonfinite = sNonFinite != 0;                   // uniform
            // slabs of consecutive groups of one segment are consecutive.  Uniform base (scalar
            // registers); the lanes add the 32-bit offset w_lane.
            const S* wchunk = Wq + (size_t)chunk_slot<FQ>(P.cpg, P.Cg, cc0) * per_slab;

            // kernel coordinates of this lane's tap, counted up with the tap groups
            int kq[ND];
            decode_tap<ND>(P, q, kq);
            T o_buf[2][ND];
            auto load_offsets_of = [&](int tgi, T* dst) {                  // offsets of tap tgi*KL + q (clamped to a legal tap)
                const S* ob = off_dg + (size_t)tgi * KL * ND * P.outV;     // uniform
                const unsigned lo = (unsigned)min(q, P.kV - 1 - tgi * KL) * ND * P.outV + pos;
#pragma unroll
                for (int a = 0; a < ND; ++a) dst[a] = Store<S>::ld((ob + (size_t)a * P.outV)[lo]);
            };
            load_offsets_of(0, o_buf[0]);

            // One tap group: geometry of this lane's (tap, position), then per group of four channels
            // eight (four) wide corner reads, the weighted corner sums and 4 * MT MFMAs.
            auto tap_group = [&](int tgi, const T* ofs) {
                const bool tap_ok = valid && tgi * KL + q < P.kV;
                // Geometry, following the reference sampler (deform3d/lib/deform_conv3d_cuda_kernel.cu:21-26,
                // 40-45,123-124) in a branch-free form: the coordinate is clamped into [0, size - 1];
                // low corner = floor, fraction toward the high corner = clamped coordinate - floor.
                // Where the reference collapses the high corner onto the low one (p <= 0,
                // p >= size - 1) the fraction is 0, so the corner one step further carries weight 0
                // and every sample uses the same eight (four) cells at fixed strides.
                bool inside = tap_ok, inhalo = true;
                T pq[ND], f[ND];
                int u[ND];
#pragma unroll
                for (int a = 0; a < ND; ++a) {
                    const int sa = slot<ND>(a);
                    const T top = (T)(P.in[sa] - 1);
                    const T pa = (ibf[a] + (T)(kq[a] * P.dil[sa])) + ofs[a];
                    T pc;
                    if constexpr (sizeof(T) == 4) pc = __builtin_amdgcn_fmed3f(pa, 0.f, top);
                    else pc = fmin(fmax(pa, (T)0), top);
                    const T fl = floor(pc);
                    pq[a] = pa;
                    f[a] = pc - fl;
                    inside = inside && fabs(pa - pc) < (T)1;                // -1 < p < size, false for NaN
                    u[a] = (int)fl - tg_.hb[a];
                    inhalo = inhalo && (unsigned)u[a] < (unsigned)(H.hext[sa] - 1);
                }
                if (halo_nonfinite) {
#pragma unroll
                    for (int a = 0; a < ND; ++a) inhalo = inhalo && pq[a] > (T)0 && pq[a] < (T)(P.in[slot<ND>(a)] - 1);
                }
                const bool near = inside && inhalo, far = inside && !inhalo;
                unsigned base;
                if constexpr (ND == 3) base = (unsigned)(__mul24(__mul24(u[0], H.hext[1]) + u[1], H.hext[2]) + u[2]);
                else base = (unsigned)(__mul24(u[0], H.hext[2]) + u[1]);
                base = near ? base : 0u;           // lanes without a sample in the halo read cell 0 and drop the value
                T cw[NC];                          // corner weights, w_l * w_h * w_w
                if constexpr (ND == 3) {
                    const T fl = f[0], gl = (T)1 - fl, fh = f[1], gh = (T)1 - fh, fw = f[2], gw = (T)1 - fw;
                    const T a00 = gl * gh, a01 = gl * fh, a10 = fl * gh, a11 = fl * fh;
                    cw[0] = a00 * gw; cw[1] = a00 * fw; cw[2] = a01 * gw; cw[3] = a01 * fw;
                    cw[4] = a10 * gw; cw[5] = a10 * fw; cw[6] = a11 * gw; cw[7] = a11 * fw;
                } else {
                    const T fh = f[0], gh = (T)1 - fh, fw = f[1], gw = (T)1 - fw;
                    cw[0] = gh * gw; cw[1] = gh * fw; cw[2] = fh * gw; cw[3] = fh * fw;
                }
                // next tap group's coordinates: KL single steps with carry, fastest axis last
#pragma unroll
                for (int st = 0; st < KL; ++st) {
                    int carry = 1;
#pragma unroll
                    for (int a = ND - 1; a > 0; --a) {
                        kq[a] += carry;
                        carry = kq[a] >= P.k[slot<ND>(a)] ? 1 : 0;
                        kq[a] = carry ? 0 : kq[a];
                    }
                    kq[0] += carry;
                }
                const V4* hp = reinterpret_cast<const V4*>(sIn) + base;
                const S* wp = wchunk + (size_t)tgi * w_tg;
                for (int grp = 0; grp < ngrp; ++grp) {
                    // this lane's weights of the group's four channels: one 16- (32-, 8-) byte load per row tile
                    typedef typename std::conditional<S16, typename Mma16<typename std::conditional<S16, S, Bf16>::type>::Vec, V4>::type A4;
                    A4 a4[MT];
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) a4[mt] = *reinterpret_cast<const A4*>(wp + (w_lane + mt * w_tile));
                    // weighted corner sum, four corners at a time (all eight in flight would cost 32
                    // registers that the 16-wavefront shape does not have)
                    // (element by element: a vector times scalar product would hold four copies of
                    // every weight)
                    T val[FQ];
                    {
                        V4 c4[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) c4[i] = hp[coff[i]];
#pragma unroll
                        for (int e = 0; e < FQ; ++e) {
                            T v = c4[0][e] * cw[0];
#pragma unroll
                            for (int i = 1; i < 4; ++i) v += c4[i][e] * cw[i];
                            val[e] = v;
                        }
                    }
                    if constexpr (ND == 3) {
                        __builtin_amdgcn_sched_barrier(0);
                        V4 c4[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) c4[i] = hp[coff[4 + i]];
#pragma unroll
                        for (int e = 0; e < FQ; ++e)
#pragma unroll
                            for (int i = 0; i < 4; ++i) val[e] += c4[i][e] * cw[4 + i];
                    }
                    if constexpr (S16) {
                        // the four channels are the four reduction elements this lane supplies to one
                        // 32x32x8 instruction (lane group q: elements 4q .. 4q + 3, its tap)
                        float b4[FQ];
#pragma unroll
                        for (int e = 0; e < FQ; ++e) b4[e] = near ? val[e] : 0.f;
                        const auto bv = Mma16<S>::pack(b4);
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt) acc[mt] = Mma16<S>::mma(a4[mt], bv, acc[mt]);
                    } else {
#pragma unroll
                        for (int e = 0; e < FQ; ++e) {
                            const T b = near ? val[e] : (T)0;
#pragma unroll
                            for (int mt = 0; mt < MT; ++mt) acc[mt] = MM::mma(a4[mt][e], b, acc[mt]);
                        }
                    }
                    hp += H.hstride;
                    wp += per_slab;
                }
                if (__any(far)) {                  // rare: some sample of this wave reaches past the halo
                    TapGeo<T, ND> t;               // the reference's corner rule on the same coordinate
                    t.inside = far;
#pragma unroll
                    for (int a = 0; a < ND; ++a) {
                        const T pa = pq[a];
                        const int l = far ? (int)pa : 0;
                        t.p[a] = pa;
                        t.lo[a] = l;
                        t.hi[a] = (pa >= (T)(P.in[slot<ND>(a)] - 1) || pa <= (T)0) ? l : l + 1;
                        t.f[a] = pa - (T)l;
                    }
                    tap_corner_idx<T, ND>(P, t);
                    const S* wf = wchunk + (size_t)tgi * w_tg;
                    for (int c = 0; c < nch; ++c) {
                        T b = 0;
                        if (far) {
                            T cc[NC];
#pragma unroll
                            for (int i = 0; i < NC; ++i) cc[i] = Store<S>::ld((chan0 + (size_t)c * P.inV)[t.idx[i]]);
                            b = interp<T, ND>(cc, t.f);
                            if constexpr (S16) b = Store<S>::ld(Store<S>::st(b));      // rounded like the samples of the halo path
                        }
                        const S* wc = wf + (size_t)(c / FQ) * per_slab + c % FQ;
                        // (one channel at a time through the float instruction: same accumulator layout)
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt) acc[mt] = MM::mma((T)Store<S>::ld(wc[w_lane + mt * w_tile]), b, acc[mt]);
                    }
                }
            };
            // two tap groups per trip: the offset registers of "this" and "next" swap roles without a
            // copy (a copy would wait for the loads a whole tap group before they are needed)
            for (int tgi = 0; tgi < ntg; tgi += 2) {
                if (tgi + 1 < ntg) load_offsets_of(tgi + 1, o_buf[1]);
                tap_group(tgi, o_buf[0]);
                if (tgi + 1 < ntg) {
                    if (tgi + 2 < ntg) load_offsets_of(tgi + 2, o_buf[0]);
                    tap_group(tgi + 1, o_buf[1]);
                }
            }
        }
    }

    if (split && whole > 0) {
        // partial sums of a unit of the last round: [split workgroup][MT * TN rows][NW * TN positions]
        T* dst = part + (size_t)pslot * (MT * TN) * (NW * TN) + wave * TN + j;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < MM::NACC; ++r) dst[(size_t)(mt * TN + MM::row(r, q)) * (NW * TN)] = acc[mt][r];
        return;
    }
    if (!valid) return;
    // unsplit: the output with bias; every unit split: a partial output tensor per cz, the bias is added when they are joined
    T* pdst = part + (size_t)cz * P.N * P.C_out * P.outV;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < MM::NACC; ++r) {
            const int m = (mchunk * MT + mt) * TN + MM::row(r, q);
            if (m < P.M) {
                const size_t at = ((size_t)n * P.C_out + g * P.M + m) * P.outV + pos;
                T v = acc[mt][r];
                if (split) pdst[at] = v;
                else {
                    if (bias) v += Store<S>::ld(bias[g * P.M + m]);
                    out[at] = Store<S>::st(v);
                }
            }
        }
}

// Joins the partial sums of the units that forward_quad_kernel split in its last round: one
// workgroup of NW * TN threads per unit and slice of JOIN_ROWS output channels, thread = position of
// the block; out = bias + the csplit partial sums, added in the order of cz.
constexpr int JOIN_ROWS = 8;
template <typename T, int ND, int MT, int NW, typename S = T>
__global__ __launch_bounds__(NW * 64) void forward_join_tail_kernel(Params P, PlanSet alts, const unsigned* __restrict__ sel,
                                                                    const T* __restrict__ part, const S* __restrict__ bias,
                                                                    S* __restrict__ out, int csplit, unsigned whole, TailSplit ts) {
    constexpr int TN = Mma<T>::TN, SLICES = MT * TN / JOIN_ROWS;
    static_assert(MT * TN % JOIN_ROWS == 0, "row slices");
    HaloPlan H;
    if (!chosen_halo(P, alts, sel, H)) return;
    if (threadIdx.x >= NW * TN) return;
    const unsigned unit = blockIdx.x / SLICES, ml0 = (blockIdx.x % SLICES) * JOIN_ROWS;
    const unsigned wg = whole + unit;
    const unsigned gm = wg % (unsigned)(P.G * P.mchunks);
    const int g = gm / P.mchunks, mchunk = gm % P.mchunks;
    TileGeo<ND> tg_;
    tile_decode<ND>(P, H, wg / (unsigned)(P.G * P.mchunks), tg_);
    int o[ND];
    unsigned pos;
    if (!tile_position<ND>(P, tg_, (int)threadIdx.x, o, pos)) return;
    size_t first = (size_t)unit * csplit;               // the unit's first partial sum
    if (ts.splitB && unit >= ts.unitsA) {
        first = (size_t)ts.unitsA * csplit + (size_t)(unit - ts.unitsA) * ts.splitB;
        csplit = ts.splitB;
    }
    const T* src = part + (first * (MT * TN) + ml0) * (NW * TN) + threadIdx.x;
    T v[JOIN_ROWS];
#pragma unroll
    for (int r = 0; r < JOIN_ROWS; ++r) v[r] = src[(size_t)r * (NW * TN)];
    for (int cz = 1; cz < csplit; ++cz) {
        T a[JOIN_ROWS];
#pragma unroll
        for (int r = 0; r < JOIN_ROWS; ++r) a[r] = src[((size_t)cz * (MT * TN) + r) * (NW * TN)];
#pragma unroll
        for (int r = 0; r < JOIN_ROWS; ++r) v[r] += a[r];
    }
#pragma unroll
    for (int r = 0; r < JOIN_ROWS; ++r) {
        const int m = mchunk * MT * TN + (int)ml0 + r;
        if (m < P.M) out[((size_t)tg_.n * P.C_out + g * P.M + m) * P.outV + pos] = Store<S>::st(bias ? v[r] + (T)Store<S>::ld(bias[g * P.M + m]) : v[r]);
    }
}

// out = bias + the sum of `parts` partial outputs of forward_quad_kernel, added in the order of the
// parts (the result does not depend on which workgroup finished first).
template <typename T>
__global__ void forward_join_partials_kernel(const T* __restrict__ part, const T* __restrict__ bias, T* __restrict__ out,
                                             int parts, size_t total, int C_out, unsigned outV) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        T v = part[i];
        for (int s = 1; s < parts; ++s) v += part[(size_t)s * total + i];
        out[i] = bias ? v + bias[(i / outV) % (size_t)C_out] : v;
    }
}

}  // namespace dcn
