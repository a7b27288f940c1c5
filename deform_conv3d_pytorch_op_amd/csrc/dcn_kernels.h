// Deformable-convolution kernels for gfx950.  All three are implicit GEMMs: the sampled column
// buffer [C_in*kV, outV] of the reference (deform3d/lib/deform_conv3d_cuda.cpp:110-148) is
// produced in registers / LDS and consumed by MFMA in the same kernel; it never reaches HBM.
//
// Lane roles.  One wavefront owns TN output positions (TN = 32 for float, 16 for double); lane
// l works on position l % TN and on reduction slot l / TN.  Offsets, corner indices and
// fractions of a (tap, position) are computed once per deformable group and reused for all of
// its channels (the reference recomputes them per channel).
#pragma once
#include "dcn_device.h"
#include <limits>
#include <type_traits>


namespace dcn {

constexpr int WG = 256;            // 4 wavefronts
constexpr int WAVES = WG / 64;

// 16-bit storage formats of the mixed-precision entry points: the tensors are widened to float
// (exactly) before the float32 kernels run and the results are rounded once, to nearest even.
struct Bf16 {       // bfloat16: the upper half of a float
    unsigned short bits;
    __device__ static inline float widen(Bf16 v) { return __uint_as_float((unsigned)v.bits << 16); }
    __device__ static inline Bf16 narrow(float f) {
        const unsigned u = __float_as_uint(f);
        Bf16 r;
        if ((u & 0x7fffffffu) > 0x7f800000u) r.bits = (unsigned short)((u >> 16) | 0x40u);      // NaN stays NaN
        else r.bits = (unsigned short)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);                  // Inf and overflow to Inf included
        return r;
    }
};
struct Fp16 {       // IEEE binary16
    _Float16 v;
    __device__ static inline float widen(Fp16 x) { return (float)x.v; }
    __device__ static inline Fp16 narrow(float f) { Fp16 r; r.v = (_Float16)f; return r; }
};
__device__ inline float offset_value(Bf16 v) { return Bf16::widen(v); }
__device__ inline float offset_value(Fp16 v) { return Fp16::widen(v); }

// Storage format of the tensors in global memory.  float / double: the arithmetic type itself.
// Bf16 / Fp16: 16-bit storage, float arithmetic; the sampled columns and the weights then meet in
// v_mfma_f32_32x32x8_bf16 / _f16 (float accumulation), a quarter of the matrix instructions.
template <typename S> struct Store { static __device__ inline S ld(S v) { return v; } static __device__ inline S st(S v) { return v; } };
template <> struct Store<Bf16> {
    static __device__ inline float ld(Bf16 v) { return Bf16::widen(v); }
    static __device__ inline Bf16 st(float v) { return Bf16::narrow(v); }
};
template <> struct Store<Fp16> {
    static __device__ inline float ld(Fp16 v) { return Fp16::widen(v); }
    static __device__ inline Fp16 st(float v) { return Fp16::narrow(v); }
};
typedef short Short4 __attribute__((ext_vector_type(4)));
typedef _Float16 Half4 __attribute__((ext_vector_type(4)));
typedef __bf16 Bfloat4 __attribute__((ext_vector_type(4)));
template <typename S> struct Mma16;
template <> struct Mma16<Bf16> {
    typedef Short4 Vec;
    static __device__ inline Vec pack(const float v[4]) {
        const Bfloat4 b = {(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};      // round to nearest even
        return __builtin_bit_cast(Short4, b);
    }
    static __device__ inline Mma<float>::Acc mma(Vec a, Vec b, Mma<float>::Acc c) { return __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a, b, c, 0, 0, 0); }
};
template <> struct Mma16<Fp16> {
    typedef Half4 Vec;
    static __device__ inline Vec pack(const float v[4]) { return Vec{(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]}; }
    static __device__ inline Mma<float>::Acc mma(Vec a, Vec b, Mma<float>::Acc c) { return __builtin_amdgcn_mfma_f32_32x32x8f16(a, b, c, 0, 0, 0); }
};

template <typename S>
__global__ void widen_kernel(const S* __restrict__ src, float* __restrict__ dst, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) dst[i] = S::widen(src[i]);
}
template <typename S>
__global__ void narrow_kernel(const float* __restrict__ src, S* __restrict__ dst, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) dst[i] = S::narrow(src[i]);
}


// ---------------------------------------------------------------------------------------------
// Weight re-layout into the workspace (tiny: the whole weight is at most a few MB).
//  forward:        Wt[g][tap][cl][m]   (m fastest, padded to Mp; cl padded to Cgp)  -> MFMA A rows = m
//  backward-data:  Wt[g][tap][m][cl]   (cl fastest, padded to Cgp; m padded to Mp)  -> MFMA A rows = channels
// Padding is zero so that reduction slots past the end contribute nothing.
template <typename T>
__global__ void relayout_weight_kernel(Params P, const T* __restrict__ W, T* __restrict__ Wt, int channel_fastest) {
    const size_t total = (size_t)P.G * P.kV * P.Mp * P.Cgp;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        int m, cl;
        size_t t;
        if (channel_fastest) { cl = i % P.Cgp; t = i / P.Cgp; m = t % P.Mp; t /= P.Mp; }
        else                 { m = i % P.Mp;  t = i / P.Mp;  cl = t % P.Cgp; t /= P.Cgp; }
        const int tap = t % P.kV, g = t / P.kV;
        T v = 0;
        if (m < P.M && cl < P.Cg) v = W[(((size_t)g * P.M + m) * P.Cg + cl) * P.kV + tap];
        Wt[i] = v;
    }
}

// Backward-data weights of the halo kernels that take CCH-channel chunks of a segment (the channels
// shared by one deformable group and one convolution group): one slab per chunk, in the order the
// lanes of a wavefront consume it, Wp[slab][pass][k][lane].  Lane (q, j) of reduction step k in MFMA
// pass `pass` holds W[m = k*KL + q][channel = first + j % CCH][tap = pass*TP + j / CCH], zero past
// M, past the last tap and past the segment, so every operand load of the kernel is one contiguous
// 64-element read (in [tap][m][channel] order the same load touches 16 separate cache lines).
// A chunk that starts at channel c0 owns slab chunk_slot(c0): increasing in c0, by at least one per
// chunk (c0 / CCH steps within a segment, one of the other terms at every segment start), so no two
// chunks share a slab; some slabs stay unused.
template <int CCH>
__host__ __device__ inline int chunk_slot(int cpg, int Cg, int c0) { return c0 / CCH + c0 / cpg + c0 / Cg; }
// The pack kernels walk over candidate chunk starts.  Where one of cpg and Cg divides the other
// (nearly every layer) the segments all have the length of the smaller and the y-th chunk start
// is known in closed form; otherwise every channel is a candidate and non-starts are skipped.
template <int CCH>
__host__ __device__ inline int chunk_candidates(int cpg, int Cg, int C_in) {
    const int seg = cpg < Cg ? cpg : Cg, big = cpg < Cg ? Cg : cpg;
    return big % seg == 0 ? C_in / seg * ((seg + CCH - 1) / CCH) : C_in;
}
template <int CCH>
__host__ __device__ inline int chunk_candidate(int cpg, int Cg, int y) {     // first channel of candidate y
    const int seg = cpg < Cg ? cpg : Cg, big = cpg < Cg ? Cg : cpg;
    if (big % seg) return y;
    const int cps = (seg + CCH - 1) / CCH;
    return y / cps * seg + y % cps * CCH;
}

// Operands of the grad-column GEMM of the fused backward kernel.  S = T: one value per lane and
// reduction step, v_mfma_f32_32x32x2_f32 / v_mfma_f64_16x16x4_f64 (KS = KL output channels per
// step).  S = Bf16 / Fp16 (T = float): four values per lane and step -- the output channels
// 8 * step + 4 * (lane / 32) + 0..3 -- for v_mfma_f32_32x32x8_bf16 / _f16, which accumulate in float
// and leave the result in the registers of the float instruction (KS = 8 output channels per step).
template <typename T, typename S> struct GcolGemm {
    static constexpr int KS = Mma<T>::KL;
    typedef T Op;
    __device__ static inline typename Mma<T>::Acc mma(Op a, Op b, typename Mma<T>::Acc c) { return Mma<T>::mma(a, b, c); }
};
template <> struct GcolGemm<float, Bf16> {
    static constexpr int KS = 8;
    typedef Mma16<Bf16>::Vec Op;
    __device__ static inline Mma<float>::Acc mma(Op a, Op b, Mma<float>::Acc c) { return Mma16<Bf16>::mma(a, b, c); }
};
template <> struct GcolGemm<float, Fp16> {
    static constexpr int KS = 8;
    typedef Mma16<Fp16>::Vec Op;
    __device__ static inline Mma<float>::Acc mma(Op a, Op b, Mma<float>::Acc c) { return Mma16<Fp16>::mma(a, b, c); }
};
// reduction steps of a weight slab's pass: a multiple of the largest operand batch
template <typename T, typename S> __host__ __device__ inline int gcol_slab_steps(int M) {
    constexpr bool S16 = !std::is_same<S, T>::value;
    return S16 ? ((M + 7) / 8 + 7) / 8 * 8 : ((M + Mma<T>::KL - 1) / Mma<T>::KL + 15) / 16 * 16;
}

// One block of 256 threads chooses the halo plan of the launches that follow (see PlanChoice).
// It reads 32 runs of 256 consecutive offset entries spread evenly over the tensor (all of a small
// one); an entry v keeps a sample inside a halo of margin m along its axis when -m <= v < m (the
// low corner floor(v) is at least -m, the high corner floor(v) + 1 at most m).  From the fraction
// e of entries beyond margin m: a sample leaves the halo with probability p = 1 - (1 - e)^nd, a
// wavefront holds such a sample with probability 1 - (1 - p)^64.
__device__ inline float offset_value(float v) { return v; }
__device__ inline float offset_value(double v) { return (float)v; }
template <typename S>
__device__ inline void choose_plan(const PlanChoice& pc, const S* __restrict__ off, size_t n) {
    __shared__ unsigned s_cnt[MAX_PLANS + 1];
    if (threadIdx.x <= MAX_PLANS) s_cnt[threadIdx.x] = 0;
    __syncthreads();
    constexpr unsigned RUN = 256, RUNS = 32;
    // counted per wavefront (ballots), so that only one lane of each adds to the shared counters
    unsigned cnt[MAX_PLANS] = {}, seen = 0;
    auto look = [&](float f, bool there) {
        seen += (unsigned)__popcll(__ballot(there));
#pragma unroll
        for (int k = 0; k < MAX_PLANS; ++k)
            cnt[k] += (unsigned)__popcll(__ballot(there && !(f >= -(float)pc.margin[k] && f < (float)pc.margin[k])));
    };
    if (n <= (size_t)RUN * RUNS) {
        for (size_t i0 = 0; i0 < n; i0 += blockDim.x) {
            const size_t i = i0 + threadIdx.x;
            const bool there = i < n;
            look(there ? offset_value(off[i]) : 0.f, there);
        }
    } else {
        // all loads of a thread in flight at once: one memory latency, not one per run
        const size_t step = (n - RUN) / (RUNS - 1);
        const bool there = threadIdx.x < RUN;
        const unsigned t = there ? threadIdx.x : 0u;
        S v[RUNS];
#pragma unroll
        for (unsigned r = 0; r < RUNS; ++r) v[r] = off[(size_t)r * step + t];
#pragma unroll
        for (unsigned r = 0; r < RUNS; ++r) look(offset_value(v[r]), there);
    }
    if ((threadIdx.x & 63) == 0) {
#pragma unroll
        for (int k = 0; k < MAX_PLANS; ++k) atomicAdd(&s_cnt[k], cnt[k]);
        atomicAdd(&s_cnt[MAX_PLANS], seen);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const float total = (float)max(s_cnt[MAX_PLANS], 1u);
        unsigned best = 0;
        float best_cost = 0.f;
        for (int k = 0; k < pc.nplans && k < MAX_PLANS; ++k) {
            const float keep = 1.f - (float)s_cnt[k] / total;             // entries inside the margin
            float in_sample = keep;
            for (int a = 1; a < pc.nd; ++a) in_sample *= keep;
            float in_wave = in_sample;
            for (int d = 0; d < 6; ++d) in_wave *= in_wave;               // ^64
            const float pf = 1.f - in_sample, pf2 = pf * pf, pf4 = pf2 * pf2;
            const float cost = pc.base[k] * (1.f + pc.far_wave * (1.f - in_wave) + pc.far_sample * pf + pc.far_steep * pf4 * pf4);
            if (k == 0 || cost < best_cost) { best = (unsigned)k; best_cost = cost; }
        }
        if (pc.global_cost > 0.f && best_cost > pc.global_cost) best = MAX_PLANS;      // no halo plan: the path through global memory
        *pc.sel = best;
    }
}

// WIDE (float, CCH = 8): row j of a pass holds (tap, channel) = (2 * (j / 16) + (j / 4) % 2,
// 4 * ((j / 8) % 2) + j % 4) instead of (j / CCH, j % CCH): the MFMA then leaves all eight channels
// of a tap in one lane (fused_row_tap / fused_row_channel).
// `bounds` (two floats, may be null) is cleared for the weight_bounds_kernel that follows.
// With pc.sel set the launch has one block more, which chooses the halo plan from the offsets.
// S = Bf16 / Fp16: Wp[slab][pass][k][lane][r] = W[m = 8 * k + 4 * q + r][...], four values per lane and step.
template <typename T, int CCH, bool WIDE = false, typename S = T>
__global__ void pack_weight_kernel(Params P, const S* __restrict__ W, S* __restrict__ Wp, float* __restrict__ bounds,
                                   PlanChoice pc, const S* __restrict__ off, size_t n_off) {
    using MM = Mma<T>;
    constexpr bool S16 = !std::is_same<S, T>::value;
    constexpr int PER = S16 ? 4 : 1;                    // values per lane and reduction step
    const unsigned pack_blocks = pc.sel ? gridDim.x - 1 : gridDim.x;
    if (blockIdx.x == pack_blocks) {
        choose_plan(pc, off, n_off);
        return;
    }
    if (bounds && blockIdx.x == 0 && threadIdx.x < 2) bounds[threadIdx.x] = 0.f;
    constexpr int TN = MM::TN, KL = MM::KL, TP = TN / CCH;
    const int npass = (P.kV + TP - 1) / TP;
    const int kst = gcol_slab_steps<T, S>(P.M);                 // operand batches are 8 or 16 (16-bit: 4 or 8) reduction steps
    const size_t per_chunk = (size_t)npass * kst * 64 * PER;
    const size_t total = (size_t)chunk_candidates<CCH>(P.cpg, P.Cg, P.C_in) * per_chunk;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)pack_blocks * blockDim.x) {
        const int c0 = chunk_candidate<CCH>(P.cpg, P.Cg, (int)(i / per_chunk));      // candidate first channel of a chunk
        const int seg_b = max(c0 / P.cpg * P.cpg, c0 / P.Cg * P.Cg);
        if ((c0 - seg_b) % CCH) continue;
        const int seg_e = min((c0 / P.cpg + 1) * P.cpg, (c0 / P.Cg + 1) * P.Cg);
        const size_t r = i % per_chunk;
        const int sub = (int)(r % PER);
        const int lane = (int)((r / PER) % 64), k = (int)((r / PER / 64) % kst), pass = (int)(r / PER / 64 / kst);
        const int q = lane / TN, j = lane % TN;
        const int jt = WIDE ? 2 * (j / 16) + (j / 4) % 2 : j / CCH, jc = WIDE ? 4 * ((j / 8) % 2) + j % 4 : j % CCH;
        const int m = S16 ? k * 8 + q * 4 + sub : k * KL + q, tap = pass * TP + jt, c = c0 + jc, g = c0 / P.Cg;
        S v = S();
        if (m < P.M && tap < P.kV && c < seg_e) v = W[(((size_t)g * P.M + m) * P.Cg + (c - g * P.Cg)) * P.kV + tap];
        Wp[(size_t)chunk_slot<CCH>(P.cpg, P.Cg, c0) * per_chunk + r] = v;
    }
}

// ---------------------------------------------------------------------------------------------
// Forward: out[n][g*M + m][pos] = sum_{cl,tap} W[g*M+m][cl][tap] * sample(in[n][g*Cg+cl], tap, pos)  (+ bias)
// replaces deformable_im2col + the per-group Sgemm (deform3d/lib/deform_conv3d_cuda.cpp:110-148,
// deform2d_double/lib/deform_conv2d_cuda.cpp:102-138).
//
// grid.x = N * tiles (a tile is WAVES*TN consecutive positions of one sample)
// grid.y = G * mchunks (a chunk is MT*TN output channels)
// The sampled value of lane (j, q) is the B operand B[k = q][col = j] of the MFMA directly; the
// A operand comes from the re-laid-out weight.
template <typename T, int ND, int MT>
__global__ __launch_bounds__(WG) void forward_kernel(Params P, const T* __restrict__ in,
                                                     const T* __restrict__ off, const T* __restrict__ Wt,
                                                     const T* __restrict__ bias, T* __restrict__ out) {
    using MM = Mma<T>;
    constexpr int TN = MM::TN, KL = MM::KL, NC = 1 << ND;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane % TN, q = lane / TN;
    const int n = blockIdx.x / P.tiles, tile = blockIdx.x % P.tiles;
    const int g = blockIdx.y / P.mchunks, mchunk = blockIdx.y % P.mchunks;

    const unsigned pos = (unsigned)(tile * WAVES + wave) * TN + j;
    const bool valid = pos < P.outV;
    const unsigned posc = valid ? pos : P.outV - 1;
    int o[ND], ib[ND];
    decode_pos<ND>(P, posc, o);
#pragma unroll
    for (int a = 0; a < ND; ++a) ib[a] = o[a] * P.stride[slot<ND>(a)] - P.pad[slot<ND>(a)];

    typename MM::Acc acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = acc_zero<T>();

    const int cg0 = g * P.Cg, cg1 = cg0 + P.Cg;
    for (int dg = cg0 / P.cpg; dg <= (cg1 - 1) / P.cpg; ++dg) {
        const int cb = max(cg0, dg * P.cpg), ce = min(cg1, (dg + 1) * P.cpg);
        const int nsteps = (ce - cb + KL - 1) / KL;
        const T* off_dg = off + ((size_t)n * P.DG + dg) * P.kV * ND * P.outV;
        for (int tap = 0; tap < P.kV; ++tap) {
            int kk[ND], kd[ND];
            decode_tap<ND>(P, tap, kk);
#pragma unroll
            for (int a = 0; a < ND; ++a) kd[a] = kk[a] * P.dil[slot<ND>(a)];
            TapGeo<T, ND> t;
            tap_setup<T, ND>(P, off_dg + (size_t)tap * ND * P.outV, posc, ib, kd, t);
            const bool live = valid && t.inside;
            // (a wave whose samples are all outside still multiplies its zero column rows: with a
            // non-finite weight the reference's GEMM turns them into NaN, and so does this)
            unsigned voff[NC];
#pragma unroll
            for (int c = 0; c < NC; ++c) voff[c] = t.idx[c] + (unsigned)q * P.inV;
            const T* chan = in + ((size_t)n * P.C_in + cb) * P.inV;                        // wave-uniform
            const T* wrow = Wt + (((size_t)g * P.kV + tap) * P.Cgp + (cb - cg0) + q) * P.Mp +
                            (size_t)mchunk * MT * TN + j;
            for (int s = 0; s < nsteps; ++s) {
                T b = 0;
                if (live && cb + s * KL + q < ce) b = sample<T, ND>(chan, voff, t.f);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[mt] = MM::mma(wrow[mt * TN], b, acc[mt]);
                chan += (size_t)KL * P.inV;
                wrow += (size_t)KL * P.Mp;
            }
        }
    }

    if (!valid) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < MM::NACC; ++r) {
            const int m = (mchunk * MT + mt) * TN + MM::row(r, q);
            if (m < P.M) {
                T v = acc[mt][r];
                if (bias) v += bias[g * P.M + m];
                out[((size_t)n * P.C_out + g * P.M + m) * P.outV + pos] = v;
            }
        }
}

// ---------------------------------------------------------------------------------------------
// Halo tiling.  A workgroup of WGH threads (1024 in the light forward variants) owns a compact
// block of output positions (tdim[0] x tdim[1] x tdim[2], one TN-wide column tile per wavefront) and stages the input neighbourhood that the
// block's samples can reach -- the "halo" -- in LDS, `cchunk` channels at a time, as channel
// planes [channel][halo voxel].  Samples whose corners all fall inside the halo are interpolated
// from LDS; the few that reach further (large offsets) fall back to global memory, so any offset
// field is handled and only the speed depends on it.
constexpr int WGH = 512;
constexpr int WAVESH = WGH / 64;
constexpr int MAX_HVOL = 6144;     // halo voxels per workgroup tile (the LDS table holds one entry each)

// Workgroups are handed to the 8 XCDs (each with its own L2) round-robin by launch order.  This
// maps the launch index of a 1-D grid to a logical index such that each XCD works through one
// contiguous range of logical indices: neighbouring tiles, and the workgroups that share a tile,
// then meet in the same L2 at about the same time.
__device__ inline unsigned xcd_contiguous(unsigned launch_idx, unsigned total) {
    constexpr unsigned XCDS = 8;
    const unsigned xcd = launch_idx % XCDS, slot = launch_idx / XCDS;
    const unsigned qq = total / XCDS, rr = total % XCDS;
    return xcd * qq + (xcd < rr ? xcd : rr) + slot;
}

template <int ND>
struct TileGeo {
    int n;              // sample
    int o0[ND];         // first output position of the tile
    int hb[ND];         // input coordinate of halo voxel (0,0,0)
};

template <int ND>
__device__ inline void tile_decode(const Params& P, const HaloPlan& H, unsigned bid, TileGeo<ND>& tg) {
    unsigned t = bid % (unsigned)P.tiles;
    tg.n = bid / (unsigned)P.tiles;
#pragma unroll
    for (int a = ND - 1; a >= 0; --a) {
        const int s = slot<ND>(a);
        const int ti = t % P.ntile[s];
        t /= P.ntile[s];
        tg.o0[a] = ti * P.tdim[s];
        tg.hb[a] = tg.o0[a] * P.stride[s] - P.pad[s] - H.mlo[s];
    }
}

// position `pt` (0 .. tile volume - 1) of the tile -> output coordinate; returns validity and the
// linear position (clamped into the volume so that offset loads of masked lanes stay legal)
template <int ND>
__device__ inline bool tile_position(const Params& P, const TileGeo<ND>& tg, int pt, int o[ND], unsigned& pos) {
    bool valid = true;
#pragma unroll
    for (int a = ND - 1; a >= 0; --a) {
        const int s = slot<ND>(a);
        const int loc = pt % P.tdim[s];
        pt /= P.tdim[s];
        int oa = tg.o0[a] + loc;
        if (oa >= P.out[s]) { valid = false; oa = P.out[s] - 1; }
        o[a] = oa;
    }
    unsigned lin = 0;
#pragma unroll
    for (int a = 0; a < ND; ++a) lin = lin * (unsigned)P.out[slot<ND>(a)] + (unsigned)o[a];
    pos = lin;
    return valid;
}

// Table of the halo: for every halo voxel its offset inside one channel of the input, or ~0u
// where the halo sticks out of the volume.  Built once per workgroup into LDS (hvol entries) so
// that staging, zeroing and flushing need no per-thread index math and no registers.
template <int ND, int WGS = WGH>
__device__ inline void halo_table(const Params& P, const HaloPlan& H, const TileGeo<ND>& tg, unsigned* __restrict__ sTab) {
    for (int v0 = threadIdx.x; v0 < H.hvol; v0 += WGS) {
        int v = v0;
        bool inb = true;
        unsigned lin = 0;
        int c[ND];
#pragma unroll
        for (int a = ND - 1; a >= 0; --a) {
            const int s = slot<ND>(a);
            c[a] = tg.hb[a] + v % H.hext[s];
            v /= H.hext[s];
            inb = inb && c[a] >= 0 && c[a] < P.in[s];
        }
#pragma unroll
        for (int a = 0; a < ND; ++a) lin = lin * (unsigned)P.in[slot<ND>(a)] + (unsigned)c[a];
        sTab[v0] = inb ? lin : ~0u;
    }
}

// Stage `nch` channels of the halo channel-interleaved, [halo voxel][CCH]: the CCH channel values of a voxel sit
// next to each other, so one wide LDS read fetches a corner of all of them (missing channels of a
// short last chunk and halo voxels outside the volume are stored as zero).
//
// Bank swizzle (float, CCH = 8).  A lane fetches four channels of a corner with one 16-byte read; with
// 32 bytes per voxel the reads of one instruction -- the same four-channel group of 64 voxels -- would
// only ever touch half of the LDS banks.  Voxel v therefore stores its four-channel group gq at
// position gq ^ (v mod groups): the same group of neighbouring voxels lands in different banks, and a
// read instruction spreads over all of them.  (Measured on 3-D layers, where the corner reads weigh
// most: the 16-channel chunks of 2-D layers lose more to the selects of the staging loop and to the
// padded halo rows than the reads gain.)
template <typename T, int CCH>
__host__ __device__ inline constexpr int swizzle_groups() { return (sizeof(T) == 4 && CCH == 8) ? CCH / 4 : 1; }
template <typename T, int CCH, int WGS, typename S = T>
__device__ inline void halo_stage_interleaved(const Params& P, const HaloPlan& H, const S* __restrict__ chan0, int nch,
                                              const unsigned* __restrict__ sTab, T* __restrict__ sIn, int* __restrict__ nonfinite) {
    constexpr int GPV = swizzle_groups<T, CCH>();
    bool bad = false;                  // a NaN or an infinity among the staged values
    for (int v = threadIdx.x; v < H.hvol; v += WGS) {
        const unsigned t = sTab[v];
        const unsigned g = t == ~0u ? 0u : t;
        T val[CCH];
#pragma unroll
        for (int c = 0; c < CCH; ++c) val[c] = Store<S>::ld(chan0[(size_t)min(c, nch - 1) * P.inV + g]);   // CCH loads in flight
        // cells outside the volume hold zero: samples in the rim read them with weight zero
#pragma unroll
        for (int c = 0; c < CCH; ++c) bad = bad || !(fabs(val[c]) <= std::numeric_limits<T>::max());
#pragma unroll
        for (int c = 0; c < CCH; ++c) val[c] = (c < nch && t != ~0u) ? val[c] : (T)0;
        if constexpr (GPV > 1) {
            const int sw = v & (GPV - 1);
#pragma unroll
            for (int gq = 0; gq < GPV; ++gq) {          // slot gq of the voxel holds group gq ^ sw
                T o4[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    T x = val[e];                        // sw == gq
#pragma unroll
                    for (int src = 0; src < GPV; ++src) x = (gq ^ sw) == src ? val[src * 4 + e] : x;
                    o4[e] = x;
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) sIn[(size_t)v * CCH + gq * 4 + e] = o4[e];
            }
        } else {
#pragma unroll
            for (int c = 0; c < CCH; ++c) sIn[(size_t)v * CCH + c] = val[c];
        }
    }
    if (bad) *nonfinite = 1;
}

// ---------------------------------------------------------------------------------------------
// Layout changes between [C][V] (channel planes, what PyTorch hands over) and [V][C]
// (channels-last, what the scatter / coordinate kernel wants so that the lanes of a wavefront
// touch consecutive addresses).  32x32 tiles through LDS; grid (ceil(V/32), ceil(C/32), N),
// block (32, 8).
template <typename T>
__global__ void to_channels_last_kernel(const T* __restrict__ src, T* __restrict__ dst, int C, unsigned V) {
    __shared__ T tile[32][33];
    const size_t base = (size_t)blockIdx.z * C * V;
    const unsigned v0 = blockIdx.x * 32;
    const int c0 = blockIdx.y * 32;
    for (int i = threadIdx.y; i < 32; i += 8) {
        const int c = c0 + i;
        const unsigned v = v0 + threadIdx.x;
        if (c < C && v < V) tile[i][threadIdx.x] = src[base + (size_t)c * V + v];
    }
    __syncthreads();
    for (int i = threadIdx.y; i < 32; i += 8) {
        const unsigned v = v0 + i;
        const int c = c0 + threadIdx.x;
        if (c < C && v < V) dst[base + (size_t)v * C + c] = tile[threadIdx.x][i];
    }
}

// dst[C][V] += src[V][C]
template <typename T>
__global__ void add_from_channels_last_kernel(const T* __restrict__ src, T* __restrict__ dst, int C, unsigned V,
                                              const unsigned* __restrict__ gate = nullptr, unsigned gate_want = 0) {
    if (gated_out(gate, gate_want)) return;
    __shared__ T tile[32][33];
    const size_t base = (size_t)blockIdx.z * C * V;
    const unsigned v0 = blockIdx.x * 32;
    const int c0 = blockIdx.y * 32;
    for (int i = threadIdx.y; i < 32; i += 8) {
        const unsigned v = v0 + i;
        const int c = c0 + threadIdx.x;
        if (c < C && v < V) tile[i][threadIdx.x] = src[base + (size_t)v * C + c];
    }
    __syncthreads();
    for (int i = threadIdx.y; i < 32; i += 8) {
        const int c = c0 + i;
        const unsigned v = v0 + threadIdx.x;
        if (c < C && v < V) dst[base + (size_t)c * V + v] += tile[threadIdx.x][i];
    }
}

// Everything the path without LDS tiling needs before its main kernel, in one launch of 256-thread
// blocks (a launch costs microseconds also when the device has chosen another path and the blocks
// return at once): blocks [0, nb_w) re-lay the weight as [g][tap][m][channel] with zero tap slabs
// behind it, blocks [nb_w, nb_w + nb_z) clear the channels-last gradient, the others transpose the
// input into its channels-last copy, 32 x 32 tiles through LDS.
template <typename T>
__global__ __launch_bounds__(256) void global_path_prepare_kernel(Params P, const T* __restrict__ W, T* __restrict__ Wt, size_t wt_pad,
                                                                  T* __restrict__ gin_cl, const T* __restrict__ in, T* __restrict__ in_cl,
                                                                  unsigned nb_w, unsigned nb_z, const unsigned* __restrict__ gate,
                                                                  unsigned gate_want) {
    if (gated_out(gate, gate_want)) return;
    const unsigned b = blockIdx.x;
    if (b < nb_w) {
        const size_t total = (size_t)P.G * P.kV * P.Mp * P.Cgp;
        for (size_t i = (size_t)b * 256 + threadIdx.x; i < total + wt_pad; i += (size_t)nb_w * 256) {
            T v = 0;
            if (i < total) {
                const int cl = i % P.Cgp;
                size_t t = i / P.Cgp;
                const int m = t % P.Mp;
                t /= P.Mp;
                const int tap = t % P.kV, g = t / P.kV;
                if (m < P.M && cl < P.Cg) v = W[(((size_t)g * P.M + m) * P.Cg + cl) * P.kV + tap];
            }
            Wt[i] = v;
        }
        return;
    }
    const size_t nelem = (size_t)P.N * P.C_in * P.inV;
    if (b < nb_w + nb_z) {
        for (size_t i = (size_t)(b - nb_w) * 256 + threadIdx.x; i < nelem; i += (size_t)nb_z * 256) gin_cl[i] = 0;
        return;
    }
    __shared__ T tile[32][33];
    const unsigned tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const unsigned vt = (P.inV + 31) / 32, ct = ((unsigned)P.C_in + 31) / 32;
    const size_t ntiles = (size_t)P.N * ct * vt;
    const unsigned nb_t = gridDim.x - nb_w - nb_z;
    for (size_t tno = b - nb_w - nb_z; tno < ntiles; tno += nb_t) {
        const unsigned v0 = (unsigned)(tno % vt) * 32, c0 = (unsigned)((tno / vt) % ct) * 32;
        const size_t base = (tno / vt / ct) * (size_t)P.C_in * P.inV;
        __syncthreads();
        for (unsigned i = ty; i < 32; i += 8) {
            const unsigned c = c0 + i, v = v0 + tx;
            if (c < (unsigned)P.C_in && v < P.inV) tile[i][tx] = in[base + (size_t)c * P.inV + v];
        }
        __syncthreads();
        for (unsigned i = ty; i < 32; i += 8) {
            const unsigned v = v0 + i, c = c0 + tx;
            if (c < (unsigned)P.C_in && v < P.inV) in_cl[base + (size_t)v * P.C_in + c] = tile[tx][i];
        }
    }
}

template <typename T>
__global__ void fill_zero_kernel(T* __restrict__ p, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0;
}

// Sum over the TN lanes that share a reduction slot (lanes l with equal l / TN).  For float the
// 16-lane rows are summed with DPP adds and the two rows of a 32-lane group are joined with a
// row broadcast, so the result is only guaranteed in the UPPER 16 lanes of each group; for
// double a shuffle butterfly leaves it in every lane.  holder(j) tells which lanes hold it.
template <int CTRL, int ROW_MASK>
__device__ inline float dpp_term(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, false));
}
__device__ inline float group_sum(float v) {
    v += dpp_term<0xB1, 0xF>(v);      // quad_perm [1,0,3,2]
    v += dpp_term<0x4E, 0xF>(v);      // quad_perm [2,3,0,1]
    v += dpp_term<0x141, 0xF>(v);     // row_half_mirror
    v += dpp_term<0x140, 0xF>(v);     // row_mirror: every lane of a 16-lane row holds the row sum
    v += dpp_term<0x142, 0xA>(v);     // row_bcast15 into rows 1 and 3: upper row of each 32-lane group
    return v;
}
__device__ inline double group_sum(double v) {
#pragma unroll
    for (int sh = 1; sh < 16; sh <<= 1) v += __shfl_xor(v, sh);
    return v;
}
template <typename T> __device__ inline bool sum_holder(int j);
template <> __device__ inline bool sum_holder<float>(int j) { return j >= 16; }
template <> __device__ inline bool sum_holder<double>(int) { return true; }

// ---------------------------------------------------------------------------------------------
// Backward to input and offset, channels-last.  Per (tap, TN positions, TN channels) the
// transposed grad-column tile
//     gcolT[pos][c] = sum_m gout[n][g*M+m][pos] * W[g*M+m][c][tap]
// is formed by MFMA (replaces the Sgemm at deform3d/lib/deform_conv3d_cuda.cpp:213-220) and lands
// with lanes along CHANNELS and registers along positions.  With input and grad-input held
// channels-last ([voxel][channel]) every corner access of the two consumers is one contiguous
// run of TN channels per lane group:
//   col2im_input  (deform3d kernel.cu:229-296, 2-D deform2d_double kernel.cu:201-238): the value
//                 is added to the 8 (4) corners with weights (w_l*w_h*w_w)*gcol by hardware float
//                 atomics on consecutive addresses;
//   col2im_offset (deform3d kernel.cu:386-483, 2-D :309-366): gcol times the derivative of the
//                 interpolation along each axis, summed over the channels of the deformable
//                 group -- a reduction across lanes -- plus, 3-D only, the out-of-range branches
//                 (:470-481), which compare the h and w coordinates against the LENGTH extent
//                 exactly like the reference.
// The geometry of a (tap, position) is computed once by the lane that owns the position and
// handed to the channel lanes through LDS.
// grid.x = N * tiles, grid.y = DG.  grad_offset gets a plain store of every element.
// SCATTER = false leaves grad-input to backward_input_halo_kernel and only writes grad_offset.
// MK > 0: the wavefront's grad_output slab (MK reduction steps of KL output channels) stays in
// registers and the weight operands of a tile are fetched in one batch; MK == 0: any M.
template <typename T, int ND, bool SCATTER, int MK>
__global__ __launch_bounds__(WG) void backward_data_kernel(Params P, const T* __restrict__ in_cl,
                                                           const T* __restrict__ off, const T* __restrict__ Wt,
                                                           const T* __restrict__ gout, T* __restrict__ gin_cl,
                                                           T* __restrict__ goff, const unsigned* __restrict__ gate = nullptr,
                                                           unsigned gate_want = 0) {
    if (gated_out(gate, gate_want)) return;
    using MM = Mma<T>;
    constexpr int TN = MM::TN, KL = MM::KL, NC = 1 << ND, NACC = MM::NACC;
    __shared__ __align__(16) unsigned sIdx[WAVES][TN][NC];   // corner voxel index * C_in
    __shared__ __align__(16) T sCw[WAVES][TN][NC];           // corner weights
    __shared__ __align__(16) T sMisc[WAVES][TN][8];          // f[ND] | oob sign[ND] at 3.. | inside flag at 6
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane % TN, q = lane / TN;
    const int n = blockIdx.x / P.tiles, tile = blockIdx.x % P.tiles;
    const int dg = blockIdx.y;

    const unsigned pos0 = (unsigned)(tile * WAVES + wave) * TN;
    const unsigned pos = pos0 + j;
    const bool valid = pos < P.outV;
    const unsigned posc = valid ? pos : P.outV - 1;
    int o[ND], ib[ND];
    decode_pos<ND>(P, posc, o);
#pragma unroll
    for (int a = 0; a < ND; ++a) ib[a] = o[a] * P.stride[slot<ND>(a)] - P.pad[slot<ND>(a)];

    const int c_lo = dg * P.cpg, c_hi = c_lo + P.cpg;
    const T* off_dg = off + ((size_t)n * P.DG + dg) * P.kV * ND * P.outV;
    T* goff_dg = goff + ((size_t)n * P.DG + dg) * P.kV * ND * P.outV;
    const T* in_n = in_cl + (size_t)n * P.inV * P.C_in;
    T* gin_n = gin_cl + (size_t)n * P.inV * P.C_in;

    // grad_output slab of this wavefront: A[row = position j][k = output channel]
    const int g_first = c_lo / P.Cg, g_last = (c_hi - 1) / P.Cg;
    T greg[MK > 0 ? MK : 1];
    auto load_slab = [&](int g) {
        const T* gq = gout + ((size_t)n * P.C_out + (size_t)g * P.M + q) * P.outV + posc;
#pragma unroll
        for (int k = 0; k < (MK > 0 ? MK : 1); ++k)
            greg[k] = (valid && k * KL + q < P.M) ? gq[(size_t)k * KL * P.outV] : (T)0;
    };
    if constexpr (MK > 0) load_slab(g_first);

    T onext[ND];
    load_offsets<T, ND>(P, off_dg, posc, onext);
    for (int tap = 0; tap < P.kV; ++tap) {
        int kk[ND], kd[ND];
        decode_tap<ND>(P, tap, kk);
#pragma unroll
        for (int a = 0; a < ND; ++a) kd[a] = kk[a] * P.dil[slot<ND>(a)];
        T ocur[ND];
#pragma unroll
        for (int a = 0; a < ND; ++a) ocur[a] = onext[a];
        if (tap + 1 < P.kV) load_offsets<T, ND>(P, off_dg + (size_t)(tap + 1) * ND * P.outV, posc, onext);
        TapGeo<T, ND> t;
        tap_setup<T, ND>(P, ocur, ib, kd, t);
        const bool live = valid && t.inside;
        T oob[3] = {0, 0, 0};
        if (ND == 3 && valid && !t.inside && !P.oob_zero) {
            const T len = (T)P.in[0];
#pragma unroll
            for (int a = 0; a < ND; ++a) oob[a] = (t.p[a] <= (T)-1) ? (T)-1 : ((t.p[a] >= len) ? (T)1 : (T)0);
        }
        const bool any_oob = oob[0] != 0 || oob[1] != 0 || oob[2] != 0;
        const bool work = __any(live || any_oob);

        __syncthreads();            // the previous tap's readers are done
        if (q == 0) {
            T cw[NC];
            if constexpr (ND == 3) {   // multiplied in the reference's order (w_l * w_h * w_w)
                const T fl = t.f[0], gl = (T)1 - fl, fh = t.f[1], gh = (T)1 - fh, fw = t.f[2], gw = (T)1 - fw;
                cw[0] = gl * gh * gw; cw[1] = gl * gh * fw; cw[2] = gl * fh * gw; cw[3] = gl * fh * fw;
                cw[4] = fl * gh * gw; cw[5] = fl * gh * fw; cw[6] = fl * fh * gw; cw[7] = fl * fh * fw;
            } else {
                const T fh = t.f[0], gh = (T)1 - fh, fw = t.f[1], gw = (T)1 - fw;
                cw[0] = gh * gw; cw[1] = gh * fw; cw[2] = fh * gw; cw[3] = fh * fw;
            }
#pragma unroll
            for (int i = 0; i < NC; ++i) {
                sIdx[wave][j][i] = t.idx[i] * (unsigned)P.C_in;
                sCw[wave][j][i] = cw[i];
            }
#pragma unroll
            for (int a = 0; a < ND; ++a) sMisc[wave][j][a] = t.f[a];
#pragma unroll
            for (int a = 0; a < 3; ++a) sMisc[wave][j][3 + a] = oob[a];
            sMisc[wave][j][6] = live ? (T)1 : (T)0;
        }
        __syncthreads();

        T ga[NACC][ND];
#pragma unroll
        for (int r = 0; r < NACC; ++r)
#pragma unroll
            for (int a = 0; a < ND; ++a) ga[r][a] = 0;

        if (work) {
            for (int g = g_first; g <= g_last; ++g) {
                const int rb = max(c_lo, g * P.Cg), re = min(c_hi, (g + 1) * P.Cg);
                const T* gb = gout + ((size_t)n * P.C_out + (size_t)g * P.M) * P.outV + posc;
                if constexpr (MK > 0) {
                    if (g_first != g_last) load_slab(g);      // several convolution groups share this deformable group
                }
                for (int c0 = rb; c0 < re; c0 += TN) {
                    typename MM::Acc d = acc_zero<T>();
                    const T* wb = Wt + (((size_t)g * P.kV + tap) * P.Mp + q) * P.Cgp + (c0 - g * P.Cg) + j;
                    if constexpr (MK > 0) {
                        T wreg[MK];                                            // B[k = m][col = channel j]
#pragma unroll
                        for (int k = 0; k < MK; ++k) wreg[k] = wb[(size_t)k * KL * P.Cgp];
                        __builtin_amdgcn_sched_barrier(0);      // keep the loads batched ahead of the MFMA chain
#pragma unroll
                        for (int k = 0; k < MK; ++k) d = MM::mma(greg[k], wreg[k], d);
                    } else {
                        const T* gq = gb + (size_t)q * P.outV;
                        for (int m0 = 0; m0 < P.M; m0 += KL) {
                            const T a = (valid && m0 + q < P.M) ? *gq : (T)0;  // A[row = position j][k = m]
                            const T b = *wb;                                   // B[k = m][col = channel j]
                            d = MM::mma(a, b, d);
                            wb += (size_t)KL * P.Cgp;
                            gq += (size_t)KL * P.outV;
                        }
                    }
                    const int c = c0 + j;
                    if (c < re) {
#pragma unroll
                        for (int r = 0; r < NACC; ++r) {
                            const int rho = MM::row(r, q);
                            const T gv = d[r];
                            const T* misc = sMisc[wave][rho];
                            if (misc[6] != (T)0) {
                                unsigned ix[NC];
                                T v[NC];
#pragma unroll
                                for (int i = 0; i < NC; ++i) ix[i] = sIdx[wave][rho][i] + (unsigned)c;
#pragma unroll
                                for (int i = 0; i < NC; ++i) v[i] = in_n[ix[i]];
                                if constexpr (ND == 3) {
                                    const T fl = misc[0], gl = (T)1 - fl, fh = misc[1], gh = (T)1 - fh,
                                            fw = misc[2], gw = (T)1 - fw;
                                    const T dl = ((v[4] - v[0]) * gw + (v[5] - v[1]) * fw) * gh +
                                                 ((v[6] - v[2]) * gw + (v[7] - v[3]) * fw) * fh;
                                    const T dh = ((v[2] - v[0]) * gw + (v[3] - v[1]) * fw) * gl +
                                                 ((v[6] - v[4]) * gw + (v[7] - v[5]) * fw) * fl;
                                    const T dw = ((v[1] - v[0]) * gh + (v[3] - v[2]) * fh) * gl +
                                                 ((v[5] - v[4]) * gh + (v[7] - v[6]) * fh) * fl;
                                    ga[r][0] += gv * dl; ga[r][1] += gv * dh; ga[r][2] += gv * dw;
                                } else {
                                    const T fh = misc[0], gh = (T)1 - fh, fw = misc[1], gw = (T)1 - fw;
                                    ga[r][0] += gv * ((v[2] - v[0]) * gw + (v[3] - v[1]) * fw);
                                    ga[r][1] += gv * ((v[1] - v[0]) * gh + (v[3] - v[2]) * fh);
                                }
                                if constexpr (SCATTER) {
#pragma unroll
                                    for (int i = 0; i < NC; ++i) atomic_add(gin_n + ix[i], sCw[wave][rho][i] * gv);
                                }
                            } else if constexpr (ND == 3) {
                                const T av = gv > 0 ? gv : -gv;
#pragma unroll
                                for (int a = 0; a < ND; ++a)      // selected, not multiplied: 0 * inf would be NaN where the reference adds nothing
                                    ga[r][a] += misc[3 + a] < (T)0 ? -av : (misc[3 + a] > (T)0 ? av : (T)0);
                            }
                        }
                    }
                }
            }
        }
        // per position: sum over the channel lanes, then the lanes that hold the sums store
        // them, lane <-> register r, i.e. position row(r, q)
#pragma unroll
        for (int a = 0; a < ND; ++a) {
            T mine = 0;
#pragma unroll
            for (int r = 0; r < NACC; ++r) {
                const T s = group_sum(ga[r][a]);
                if ((j % 16) == r) mine = s;
            }
            const int r_mine = j % 16;
            if (sum_holder<T>(j) && r_mine < NACC && (TN == 32 || j < 16)) {
                const unsigned p_out = pos0 + MM::row(r_mine, q);
                if (p_out < P.outV) goff_dg[((size_t)tap * ND + a) * P.outV + p_out] = mine;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// LDS accumulation cell of the privatised scatter.  LDS float atomics (ds_add_f32) are an order
// of magnitude slower than LDS integer atomics on gfx950, so float contributions are summed as
// 64-bit fixed point: value * 2^e rounded to an integer and added with ds_add_u64.  The exponent
// e is chosen per workgroup and convolution group from a bound on the largest possible term
// (8 * max|W| * max_pos sum_m |grad_output|), leaving 2^17 terms of headroom below 2^47; the
// integer sum is exact, so the result is rounded once when the cell is flushed.  A bound that is
// not finite (NaN or infinity in grad_output or the weights) has no exponent: such a workgroup
// sends every contribution through the global float atomics of the far path instead, which
// propagate NaN and infinity like the reference's atomicAdd.  double keeps a
// floating cell (ds_add_f64): its 1e-10 tolerance is tighter than the fixed-point grid.
template <typename T> struct LdsCell;
template <> struct LdsCell<float> {
    typedef unsigned long long type;
    static constexpr double MAGIC = 6755399441055744.0;     // 1.5 * 2^52: low mantissa bits = integer value
    // The bit pattern of MAGIC + x is the pattern of MAGIC plus the integer x (|x| < 2^51), and the
    // pattern of MAGIC is zero in its low 48 bits: the raw patterns are summed and, whatever the
    // number of terms a cell receives, its low 48 bits hold the sum of the integers modulo 2^48.
    __device__ static inline void add(type* p, double w, double gv_scaled) {
        const double d = __builtin_fma(w, gv_scaled, MAGIC);
        (void)__hip_atomic_fetch_add(p, (type)__double_as_longlong(d), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    __device__ static inline double pre(float gv, double scale) { return (double)gv * scale; }
    __device__ static inline float value(type c, double inv_scale) {
        return (float)((double)((long long)(c << 16) >> 16) * inv_scale);      // sign-extended low 48 bits
    }
    // Two channels in one cell: signed 32-bit integers a (low half) and b (high half) are added as
    // the single 64-bit number b * 2^32 + a, i.e. with b lowered by one where a is negative, so
    // that any number of terms sums exactly in both halves as long as each half's sum fits 32
    // bits (the caller scales the terms accordingly).
    // The terms are turned into integers by a float FMA against 1.5 * 2^23, whose result carries the
    // rounded product in its low mantissa bits (|term| < 2^22, which the caller's scale ensures).
    static constexpr float MAGIC32 = 12582912.f;             // 1.5 * 2^23, bit pattern 0x4B400000
    __device__ static inline void add2(type* p, float w, float g0_scaled, float g1_scaled) {
        // one 64-bit subtraction strips the constant from both halves; its borrow out of the low half
        // (exactly when a is negative) is the lowering of b by one
        typedef float F2 __attribute__((ext_vector_type(2)));
        const F2 t = {__builtin_fmaf(w, g0_scaled, MAGIC32), __builtin_fmaf(w, g1_scaled, MAGIC32)};
        const type raw = __builtin_bit_cast(type, t);
        (void)__hip_atomic_fetch_add(p, raw - 0x4B4000004B400000ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    __device__ static inline void value2(type c, double inv_scale, float& v0, float& v1) {
        const int a = (int)(unsigned)c;
        const int b = (int)(unsigned)(c >> 32) - (a >> 31);        // undo the borrow of a negative low half
        v0 = (float)((double)a * inv_scale);
        v1 = (float)((double)b * inv_scale);
    }
};
template <> struct LdsCell<double> {
    typedef double type;
    __device__ static inline void add(type* p, double w, double gv) {
        (void)__hip_atomic_fetch_add(p, w * gv, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    __device__ static inline double pre(double gv, double) { return gv; }
    __device__ static inline double value(type c, double) { return c; }
};

// max |w| over a small tensor (used for the fixed-point exponent), NaN if any element is NaN.  Each
// workgroup reduces a strided share and joins the result with an integer atomic max: non-negative
// floats order like their bit patterns.  `out` must hold 0 beforehand.
template <typename T>
__global__ void absmax_kernel(const T* __restrict__ w, size_t n, float* __restrict__ out) {
    __shared__ float red[256];
    // maxima are taken on the bit patterns: |NaN| has the largest pattern, so a NaN survives (fmaxf drops it)
    unsigned m = 0u;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        m = max(m, __float_as_uint(fabsf((float)w[i])));
    unsigned* redu = reinterpret_cast<unsigned*>(red);
    redu[threadIdx.x] = m;
    __syncthreads();
    for (int sft = blockDim.x / 2; sft > 0; sft >>= 1) {
        if ((int)threadIdx.x < sft) redu[threadIdx.x] = max(redu[threadIdx.x], redu[threadIdx.x + sft]);
        __syncthreads();
    }
    if (threadIdx.x == 0) atomicMax(reinterpret_cast<unsigned*>(out), redu[0]);
}

// out[0] = max |w| and out[1] = max over the weight's (input channel, tap) columns of the Euclidean
// norm over the output channels of one convolution group, NaN if any element is NaN: |grad column|
// <= that norm times the norm of grad_output over the output channels at the position
// (Cauchy-Schwarz).  W is [G*M][Cg][kV]; grid (ceil(Cg*kV / 64), G); joined like absmax_kernel.
// `out` must hold two zeros beforehand.
template <typename T>
__global__ __launch_bounds__(512) void weight_bounds_kernel(const T* __restrict__ w, int M, size_t cols, float* __restrict__ out) {
    // workgroup = 64 neighbouring columns of one group (blockIdx.y) x 8 slices of its rows
    __shared__ float part[8][64];
    __shared__ unsigned amax[8];
    const int cx = threadIdx.x & 63, sl = threadIdx.x >> 6;
    const size_t col = (size_t)blockIdx.x * 64 + cx;
    float ss = 0.f;
    unsigned am = 0u;
    if (col < cols) {
        const T* p = w + (size_t)blockIdx.y * M * cols + col;
#pragma unroll 8
        for (int r = sl; r < M; r += 8) {
            const float v = offset_value(p[(size_t)r * cols]);
            ss += v * v;
            am = max(am, __float_as_uint(fabsf(v)));
        }
    }
    for (int sh = 1; sh < 64; sh <<= 1) am = max(am, (unsigned)__shfl_xor((int)am, sh));
    part[sl][cx] = ss;
    if (cx == 0) amax[sl] = am;
    __syncthreads();
    if (sl == 0) {
#pragma unroll
        for (int k = 1; k < 8; ++k) { ss += part[k][cx]; am = max(am, amax[k]); }
        unsigned m = __float_as_uint(fabsf(sqrtf(ss)));       // NaN keeps the largest pattern
        for (int sh = 1; sh < 64; sh <<= 1) m = max(m, (unsigned)__shfl_xor((int)m, sh));
        if (cx == 0) {
            atomicMax(reinterpret_cast<unsigned*>(out), am);          // out[0] = max |w|
            atomicMax(reinterpret_cast<unsigned*>(out) + 1, m);       // out[1] = largest column norm
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Backward to input with the scatter privatised in LDS (col2im_input of the reference,
// deform3d kernel.cu:229-296 / deform2d_double kernel.cu:201-238, fed by the grad-column GEMM of
// deform3d/lib/deform_conv3d_cuda.cpp:213-220).
//
// Same halo tiling as forward_quad_kernel, but the LDS planes hold the partial grad-input of CCH
// channels over the halo of the workgroup's position block (cells: see LdsCell).  The rows of
// one MFMA tile are (tap, channel) pairs -- TP = TN / CCH taps of the CCH channels -- so a pass
// of ceil(M / KL) MFMAs yields the grad-column values gcol[c][tap][pos] of TP taps at once with
// lanes along positions.  Each lane then walks its registers: per tap slot it derives the corner
// cells and weights of its position once, per channel it adds (w_l*w_h*w_w)*gcol to the 8 (4)
// corners with LDS integer atomics.  The MFMAs of the next pass are issued between those steps.
// After all taps the planes are added to grad_input with one hardware float atomic per touched
// halo voxel -- about 1/30 of the global atomics of a direct scatter.  Samples that reach past
// the halo use global atomics directly, in a pass of their own.
// 1-D grid: `whole` workgroups with one (tile, deformable group) item each, then csplit
// workgroups for each remaining item; dynamic LDS = CCH * hstride * 8 + hvol * 4 bytes.
// COORD = true additionally stages the same CCH input channels over the halo (float planes) and
// computes grad_offset in the same pass over the grad-column values (col2im_offset of the
// reference, deform3d kernel.cu:386-483 incl. the out-of-range branches :470-481, 2-D
// deform2d_double kernel.cu:309-366): per (tap, position) the derivative of the interpolation
// along each axis times gcol, summed over the chunk's channels, accumulated into grad_offset
// chunk after chunk (float atomics on a zero-filled buffer, or the first chunk stores and the
// others add in place).  dynamic LDS then adds CCH * hstride * sizeof(T).
// BREG = true (host: at most 32 * BS reduction steps, i.e. M <= 64 * BS for float) keeps this lane's
// grad_output values -- the B operand, the same for every tap and channel chunk -- in registers;
// the first 32 steps of a pass ride on the tap slots of the pass before, the others (BS = 2) run ahead of them.
// NW wavefronts per workgroup (8; 4 where only a smaller block of positions has a halo that fits).
// HS > 0 fixes the plane stride at compile time (the host then plans with hstride = HS): the plane
// of a channel becomes an immediate offset of the LDS instructions instead of address arithmetic.
// PACKW: the weights come in the per-chunk lane order of pack_weight_kernel instead of
// [g][tap][m][channel].
// CCH = 16 (float, 2-D layers whose halo leaves room for 16 channel planes): two taps per pass, so the
// nine taps of a 3x3 kernel take 5 passes per 16 channels instead of 6, with half as many chunks to
// zero, stage and flush; a lane then holds eight channels of each of the two taps (0..3 and 8..11 in
// lane group 0, 4..7 and 12..15 in lane group 1) and walks them as two tap slots.
// PAIR (float only): the cells hold two channels each as 32-bit fixed point (LdsCell<float>::add2):
// half the LDS atomics and two thirds of the LDS bytes per channel.  The terms are scaled such
// that (positions of the block x taps) of the largest possible one -- all that a cell can receive
// -- still fit 31 bits; the host allows it only while that leaves enough bits below that term.
// wmax[1] then holds the largest column norm of the weight (colnorm_max_kernel).
// S: storage format of input, offset, weight and grad_output (Bf16 / Fp16 with T = float: the grad-column
// GEMM then runs on the 16-bit matrix instructions, see GcolGemm; requires BREG and PACKW); the
// gradients are written as T.
template <typename T, int ND, int CCH, bool COORD, bool BREG, int HS, int NW, bool PACKW = false, bool PAIR = false, int BS = 1,
          int HE1 = 0, int HE2 = 0, typename S = T>
__global__ __launch_bounds__(NW * 64) void backward_input_halo_kernel(Params P, PlanSet alts, const unsigned* __restrict__ sel,
                                                                  const S* __restrict__ in,
                                                                  const S* __restrict__ off,
                                                                  const S* __restrict__ Wt,
                                                                  const S* __restrict__ gout,
                                                                  const float* __restrict__ wmax,
                                                                  T* __restrict__ gin, T* __restrict__ goff, int csplit,
                                                                  unsigned whole, int goff_atomic) {
    HaloPlan H;
    if (!chosen_halo(P, alts, sel, H)) return;          // another launch runs the chosen plan
    using MM = Mma<T>;
    using Cell = typename LdsCell<T>::type;
    constexpr int TN = MM::TN, KL = MM::KL, NC = 1 << ND, NACC = MM::NACC;
    constexpr bool S16 = !std::is_same<S, T>::value;
    using GG = GcolGemm<T, S>;
    using Op = typename GG::Op;                         // what a lane supplies to one reduction step
    constexpr int KS = GG::KS;                          // output channels per reduction step
    static_assert(!S16 || (BREG && PACKW && sizeof(T) == 4), "16-bit operands: packed weights, grad_output in registers");
    constexpr int TP = TN / CCH;                        // taps per MFMA pass
    // WIDE (paired cells, 8-channel chunks): the weight rows are ordered such that a lane receives
    // all eight channels of a tap -- lane group q the taps q and 2 + q of a pass -- instead of four
    // channels of each of four taps, with the other four in the other lane group: the geometry of a
    // (tap, position) is then worked out once per eight channels, not once per lane group.
    constexpr bool WIDE = PAIR && CCH == 8 && BREG;      // (with the grad_output operand in registers: measured slower without)
    // (16-channel chunks, float: two taps per pass, a lane holds eight channels of each -- 0..3 and 8..11 or 4..7 and 12..15)
    constexpr int RPS = (WIDE || CCH == 16) ? 8 : (MM::row(1, 0) - MM::row(0, 0) == 1) ? 4 : CCH / 4;   // registers that share a tap
    constexpr int NS = NACC / RPS;                      // tap slots per lane and pass
    // (tap of the pass, channel of the chunk) behind accumulator register r of lane group qq
    auto row_tap = [](int r, int qq) { return WIDE ? 2 * (r / 8) + qq : MM::row(r, qq) / CCH; };
    auto row_ch = [](int r, int qq) { return WIDE ? r % 8 : MM::row(r, qq) % CCH; };
    static_assert(TN % CCH == 0 && CCH % 4 == 0 && NACC % RPS == 0, "unsupported channel chunk");
    static_assert(!PAIR || (sizeof(T) == 4 && RPS % 2 == 0), "paired cells are a float32 layout");
    constexpr int CPL = PAIR ? CCH / 2 : CCH;           // cell planes
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int hs = HS ? HS : H.hstride;
    // HE1, HE2 > 0 fix the two inner halo extents at compile time (the host then launches this
    // instantiation only for plans with exactly these extents): the distances between the corners of a
    // sample become immediate offsets of the LDS instructions instead of per-corner address arithmetic
    const int he1 = HE1 ? HE1 : H.hext[1], he2 = HE2 ? HE2 : H.hext[2];
    Cell* sG = reinterpret_cast<Cell*>(smem_raw);                                       // [CPL][hstride]
    T* sIn = reinterpret_cast<T*>(sG + (size_t)CPL * hs);                               // [hstride][CCH] if COORD: channels of a voxel side by side
    unsigned* sTab = reinterpret_cast<unsigned*>(sIn + (COORD ? (size_t)CCH * hs : 0));   // [hvol]
    constexpr int WGS = NW * 64;                        // threads per workgroup
    __shared__ float sRed[NW], sSum[NW], sAmax[NW];
    __shared__ int sNonFinite;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane % TN, q = lane / TN;
    // Work items are (tile, deformable group) pairs.  The first `whole` workgroups of the launch take
    // one item each; every later item is shared by csplit workgroups, of which workgroup cz takes
    // every csplit-th channel chunk: finer work at the end of the launch fills the last, ragged
    // round of workgroups.  The grad_offset contributions of the channel chunks of a shared item meet
    // through float atomics on a zero-filled buffer; the single owner of an item stores the first
    // chunk's values and then the running sum (or uses the atomics too: goff_atomic = 1).
    unsigned item;
    int cz = 0, cs = 1;
    if (blockIdx.x < whole) item = xcd_contiguous(blockIdx.x, whole);
    else {
        const unsigned r = xcd_contiguous(blockIdx.x - whole, gridDim.x - whole);
        cs = csplit;
        item = whole + r / (unsigned)cs;
        cz = r % (unsigned)cs;
    }
    const unsigned nt = (unsigned)P.N * P.tiles;
    const int dg = item / nt;
    // an item that several workgroups share needs the atomics (the host has zero-filled grad_offset);
    // the only owner of an item stores the running sum over its chunks instead, unless the host asks for
    // atomics there as well (goff_atomic: layers with so few grad_offset elements that the atomics cost
    // less than the loads of the running sum)
    goff_atomic = cs > 1 ? 1 : goff_atomic;

    TileGeo<ND> tg;
    tile_decode<ND>(P, H, item % nt, tg);
    const int n = tg.n;
    int o[ND], ib[ND];
    unsigned pos;
    const bool valid = tile_position<ND>(P, tg, wave * TN + j, o, pos);
#pragma unroll
    for (int a = 0; a < ND; ++a) ib[a] = o[a] * P.stride[slot<ND>(a)] - P.pad[slot<ND>(a)];
    halo_table<ND, WGS>(P, H, tg, sTab);                  // visible after the first barrier below
    // o * stride - pad of this lane's position as T: the integer part of a sampling coordinate is
    // (T)(that + tap * dilation), a sum of two small integers that is exact in T as well
    T ibf[ND];
#pragma unroll
    for (int a = 0; a < ND; ++a) ibf[a] = (T)ib[a];

    const int c_lo = dg * P.cpg, c_hi = c_lo + P.cpg;
    const S* off_dg = off + ((size_t)n * P.DG + dg) * P.kV * ND * P.outV;
    T* goff_dg = goff + ((size_t)n * P.DG + dg) * P.kV * ND * P.outV;
    bool first_chunk = true;                        // grad_offset without atomics: the first channel chunk stores, later ones add
    int chunk_no = 0;
    // this lane's row of the A operand: (tap slot, channel) = (j / CCH, j % CCH)
    const int a_tl = j / CCH, a_c = j % CCH;
    const unsigned a_off = PACKW ? (unsigned)lane : ((unsigned)a_tl * P.Mp + q) * P.Cgp + a_c;      // lane offset inside a tap group's weight slabs

    for (int g = c_lo / P.Cg; g <= (c_hi - 1) / P.Cg; ++g) {
        const int rb = max(c_lo, g * P.Cg), re = min(c_hi, (g + 1) * P.Cg);
        // wave-uniform base (scalar registers) + 32-bit lane offset of the B operand grad_output[m][pos]
        constexpr int AB = ((WIDE || CCH == 16) ? 16 : 8) / (S16 ? 2 : 1);      // reduction steps per operand batch (NS * AB ride on a pass: 64 output channels, 16-bit 128)
        const S* gbase = gout + ((size_t)n * P.C_out + (size_t)g * P.M) * P.outV;
        const unsigned b_off = (unsigned)q * P.outV + pos;
        const size_t gstep = (size_t)KS * P.outV;
        // Reduction step k of this lane reads grad_output[k * KL + q][pos]: the row base advances in
        // scalar registers, clamped at the last real step (the further steps of a batch meet zero
        // weight rows and re-read that step; a lane whose row of the last step lies past M reads
        // row q = 0 of it, again against a zero weight row), and the lane adds a 32-bit byte
        // offset, so that a load costs a few scalar instructions and one select instead of 64-bit
        // address arithmetic per lane.  Lanes outside the volume read a clamped position (their
        // columns are never used).  No load is masked: a masked load becomes a conditional one,
        // issued alone with a full wait behind it.
        const int klast = (P.M + KS - 1) / KS - 1;
        const unsigned b_byte = b_off * (unsigned)sizeof(T);
        const unsigned b_byte_last = (klast * KL + q < P.M ? b_off : pos) * (unsigned)sizeof(T);
        Op b_reg[BREG ? NS * AB * BS : 1];
        float sabs = 0.f;                           // sum_m |grad_output| of this lane's position (its q share); PAIR: of the squares
        float amax = 0.f;                           // PAIR: largest |grad_output| seen (squares of tiny values underflow)
        if constexpr (S16) {
            // four output channels per lane and step: rows 8 * k + 4 * q + r of grad_output at this lane's
            // position; rows past M (last step only: zero weights there) re-read row M - 1
            int kl = klast;
            asm volatile("" : "+s"(kl));
            unsigned row_off[4], row_off_last[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                row_off[r] = ((unsigned)(4 * q + r) * P.outV + pos) * (unsigned)sizeof(S);
                const int rl = min(kl * 8 + 4 * q + r, P.M - 1) - kl * 8;
                row_off_last[r] = ((unsigned)rl * P.outV + pos) * (unsigned)sizeof(S);
            }
            const char* gk = reinterpret_cast<const char*>(gbase);
#pragma unroll
            for (int k = 0; k < NS * AB * BS; ++k) {
                float g4[4];
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    g4[r] = Store<S>::ld(*reinterpret_cast<const S*>(gk + (k >= kl ? row_off_last[r] : row_off[r])));
                gk += k < kl ? gstep * sizeof(S) : (size_t)0;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const bool counts = valid && k <= kl && k * 8 + 4 * q + r < P.M;
                    sabs += counts ? (PAIR ? g4[r] * g4[r] : fabsf(g4[r])) : 0.f;
                    if constexpr (PAIR) amax = counts ? fmaxf(amax, fabsf(g4[r])) : amax;
                }
                b_reg[k] = Mma16<S>::pack(g4);          // (exact: the values are 16-bit already)
            }
        } else if constexpr (BREG) {
            // held unmasked (rows past M meet zero weight rows, columns outside the volume are never
            // used): a masked load becomes a conditional one, issued alone with a full wait behind it
            // (the last step passes through an empty asm: the per-step selects derived from it are
            // then computed here, not hoisted out of the group loop into registers that stay live
            // through the whole kernel)
            int kl = klast;
            asm volatile("" : "+s"(kl));
            const char* gk = reinterpret_cast<const char*>(gbase);
#pragma unroll
            for (int k = 0; k < NS * AB * BS; ++k) {
                b_reg[k] = *reinterpret_cast<const T*>(gk + (k >= kl ? b_byte_last : b_byte));
                gk += k < kl ? gstep * sizeof(T) : (size_t)0;
            }
#pragma unroll
            for (int k = 0; k < NS * AB * BS; ++k) {
                const float bk = (float)b_reg[k];
                const bool counts = valid && (k < kl || (k == kl && kl * KL + q < P.M));
                sabs += counts ? (PAIR ? bk * bk : fabsf(bk)) : 0.f;
                if constexpr (PAIR) amax = counts ? fmaxf(amax, fabsf(bk)) : amax;
            }
        } else {
            // unconditional loads, eight in flight, masked when they are summed (a masked load
            // becomes a conditional one that is waited for on its own)
            const char* gk = reinterpret_cast<const char*>(gbase);
            for (int k0 = 0; k0 <= klast; k0 += AB) {
                T bv[AB];
#pragma unroll
                for (int k = 0; k < AB; ++k) {
                    bv[k] = *reinterpret_cast<const T*>(gk + (k0 + k >= klast ? b_byte_last : b_byte));
                    gk += k0 + k < klast ? gstep * sizeof(T) : (size_t)0;
                }
#pragma unroll
                for (int k = 0; k < AB; ++k) {
                    const int kk_ = k0 + k;
                    const float bk = (float)bv[k];
                    const bool counts = valid && (kk_ < klast || (kk_ == klast && klast * KL + q < P.M));
                    sabs += counts ? (PAIR ? bk * bk : fabsf(bk)) : 0.f;
                    if constexpr (PAIR) amax = counts ? fmaxf(amax, fabsf(bk)) : amax;
                }
            }
        }
        // fixed-point exponent of this (workgroup, convolution group): terms are bounded by
        // 8 * max|W| * max_pos sum_m |grad_output|
#pragma unroll
        for (int sh = TN; sh < 64; sh <<= 1) sabs += __shfl_xor(sabs, sh);
        // maxima on the bit patterns (sabs >= 0 or NaN): a NaN has the largest pattern and survives
        unsigned sbits = __float_as_uint(fabsf(sabs));
#pragma unroll
        for (int sh = 1; sh < TN; sh <<= 1) sbits = max(sbits, (unsigned)__shfl_xor((int)sbits, sh));
        // paired cells: also the sum over the block's positions of the norm of grad_output over the
        // output channels (every lane of a position holds its full sum of squares by now)
        float nsum = PAIR ? sqrtf(sabs) : 0.f;
        if constexpr (PAIR) {
#pragma unroll
            for (int sh = 1; sh < TN; sh <<= 1) nsum += __shfl_xor(nsum, sh);
#pragma unroll
            for (int sh = 1; sh < 64; sh <<= 1) amax = fmaxf(amax, __shfl_xor(amax, sh));
        }
        __syncthreads();
        if (lane == 0) { sRed[wave] = __uint_as_float(sbits); sSum[wave] = nsum; sAmax[wave] = amax; }
        __syncthreads();
        unsigned smaxb = 0u;
        float ssum = 0.f, gmax = 0.f;
#pragma unroll
        for (int w8 = 0; w8 < NW; ++w8) { smaxb = max(smaxb, __float_as_uint(sRed[w8])); ssum += sSum[w8]; gmax = fmaxf(gmax, sAmax[w8]); }
        int ex = 0;
        // paired cells: |term| <= largest column norm of W x largest norm of grad_output over the
        // output channels (0.1 % slack for the rounding of those two and of the MFMA sums)
        const float bound = PAIR ? 1.001f * wmax[1] * sqrtf(__uint_as_float(smaxb)) : 8.f * wmax[0] * __uint_as_float(smaxb);
        // paired cells: all that one cell can receive.  A (tap, position) spreads at most |grad column| over
        // its corners (their weights add up to one), so a cell's terms add up to at most the sum over the
        // block's positions and the taps of that bound -- far less than (number of terms) x (largest term)
        // when a few positions carry most of grad_output
        const float bound_cell = PAIR ? 1.001f * wmax[1] * (float)P.kV * ssum : 0.f;
        // the LDS cells need a finite bound; without one this workgroup scatters through the far path
        // (float cells need the exponent; and with either cell type a corner that carries weight zero
        // would receive 0 * inf = NaN where the reference adds nothing)
        // (and a block whose grad_output is so small that its squares underflow: the bound is then not
        // trustworthy, and the workgroup takes the far path too rather than rounding its gradient away)
        const bool cells_ok = bound < 3.0e38f && bound_cell < 3.0e38f && !(PAIR && gmax > 0.f && gmax < 1e-18f);            // false for NaN
        if (bound > 0.f && bound < 3.0e38f) (void)frexpf(bound, &ex);
        double scale = ldexp(1.0, 30 - ex), inv_scale = ldexp(1.0, ex - 30);
        float scale32 = 1.f;
        if constexpr (PAIR) {
            // a single term stays below 2^22 (the float conversion of add2) and all the terms a cell can
            // receive together below 2^31 (their roundings, half a unit each for at most NW * TN * kV
            // terms, fit the one per cent of slack)
            if (bound > 0.f && cells_ok) {
                const double s_term = 4194304.0 / (double)bound;
                const double s_cell = bound_cell > 0.f ? 2147483648.0 / (double)bound_cell : s_term;
                scale = 0.99 * (s_term < s_cell ? s_term : s_cell);
            } else
                scale = 1.0;
            scale32 = (float)(scale < 1e30 ? scale : 1e30);       // (a denormal bound: keep the scale a finite float)
            scale = (double)scale32;                 // the flush divides by exactly what the terms were multiplied with
            inv_scale = 1.0 / scale;
        }

        for (int cc0 = rb; cc0 < re; cc0 += CCH) {
            if ((chunk_no++) % cs != cz) continue;          // another workgroup's chunk (uniform)
            const int nch = min(CCH, re - cc0);
            if (threadIdx.x == 0) sNonFinite = 0;
            __syncthreads();                        // the previous chunk's flush is done
            for (int c = 0; c < (PAIR ? (nch + 1) / 2 : nch); ++c)
                for (int v = threadIdx.x; v < H.hvol; v += WGS) sG[c * hs + v] = 0;      // all-zero bits in either cell type
            if constexpr (COORD) halo_stage_interleaved<T, CCH, WGS, S>(P, H, in + ((size_t)n * P.C_in + cc0) * P.inV, nch, sTab, sIn, &sNonFinite);
            __syncthreads();
            // Non-finite input values in this halo: the branch-free sampler reads the cell next to a
            // collapsed corner with weight 0, and 0 * inf would be NaN where the reference never
            // touches that voxel (deform3d/lib/deform_conv3d_cuda_kernel.cu:24-26).  Samples in the
            // collapse zones (p <= 0 or p >= size - 1 on some axis) then take the far path, which
            // follows the reference's corner rule.
            const bool halo_nonfinite = COORD && sNonFinite != 0;          // uniform

            // Grad-column tile of a pass: row i = (tap tap0 + i / CCH, channel cc0 + i % CCH); taps past
            // the last one read zero padding (or rows that are ignored below).  The MFMAs of pass p+1
            // are issued between the tap slots of pass p, a few per accumulator register walked, so
            // the matrix pipe works behind the vector work of the scatter instead of before it.
            // Operands arrive in batches of AB reduction steps, loaded one tap slot ahead of use.
            constexpr int MPR = AB / RPS;                              // MFMAs per accumulator register walked
            const int ksteps = (P.M + KS - 1) / KS;
            // (weights are addressed in operands: one value, or with 16-bit storage four values, per lane and step)
            const Op* Wo = reinterpret_cast<const Op*>(Wt);
            const size_t wstep = PACKW ? (size_t)64 : (size_t)KL * P.Cgp;
            const size_t wpass = PACKW ? (size_t)gcol_slab_steps<T, S>(P.M) * 64 : (size_t)TP * P.Mp * P.Cgp;   // weights of one pass
            const Op* wchunk = PACKW ? Wo + (size_t)chunk_slot<CCH>(P.cpg, P.Cg, cc0) * ((P.kV + TP - 1) / TP) * wpass
                                     : Wo + ((size_t)g * P.kV * P.Mp) * P.Cgp + (cc0 - g * P.Cg);      // uniform; lanes add a_off
            // (k0 passes through an empty asm: what is derived from it is then computed where it is
            // used instead of being hoisted out of the loops into hundreds of long-lived registers)
            auto load_batch = [&](Op* a_nx, Op* b_nx, const Op* wp, int k0) {      // rows past M are zero padding
                asm volatile("" : "+s"(k0));
                const Op* wb = wp + (size_t)k0 * wstep;                // one 64-bit product per batch; the row offsets below are loop invariants
                const char* gk = reinterpret_cast<const char*>(gbase + (size_t)min(k0, klast) * gstep);
#pragma unroll
                for (int k = 0; k < AB; ++k) {
                    a_nx[k] = (wb + (unsigned)k * (unsigned)wstep)[a_off];
                    if constexpr (!BREG) {
                        b_nx[k] = *reinterpret_cast<const Op*>(gk + (k0 + k >= klast ? b_byte_last : b_byte));
                        gk += k0 + k < klast ? gstep * sizeof(T) : (size_t)0;
                    }
                }
            };
            // steps [k_begin, ksteps) of one pass in a software-pipelined loop of their own: the whole
            // first pass, and what the tap slots cannot take when M is large
            // (two operand sets that swap roles from batch to batch, two batches per loop trip: copying
            // "next" into "current" costs 2 * AB register moves per batch whenever the register
            // allocator cannot merge the sets, on the same issue port as the MFMAs)
            auto gemm_tail = [&](typename MM::Acc& dd, const Op* wp, int k_begin) {
                Op a_s[2][AB], b_s[2][AB];
                load_batch(a_s[0], b_s[0], wp, k_begin);
                int k0 = k_begin;
                if (PACKW && ksteps - k_begin >= 96) {
                    // Long reductions (M >= 192 float): the next batch is requested in the same block
                    // as this batch's MFMAs (past the last step the padded slab's last batch is read
                    // again) and the scheduler is told to deal the address arithmetic and the loads out
                    // between the MFMAs.  The wavefronts of a workgroup run in step, so a separate load
                    // phase leaves the matrix pipe idle in all of them at once.  (Short reductions lose
                    // more to the one redundant batch than they gain.)
                    const int k_last = (int)(wpass / 64) - AB;
                    // Batches all of whose steps are real ones for every lane need no clamping of the
                    // grad_output rows: two scalar adds per load instead of a dozen scalar instructions,
                    // which a wavefront has to issue between two MFMAs.
                    const int kfast_end = P.M % KL == 0 ? klast + 1 : klast;      // steps [0, kfast_end) load without a clamp
                    auto load_fast = [&](Op* a_nx, Op* b_nx, int k0f) {
                        asm volatile("" : "+s"(k0f));
                        const Op* wb = wp + (size_t)k0f * wstep;
                        const char* gk = reinterpret_cast<const char*>(gbase + (size_t)k0f * gstep);
#pragma unroll
                        for (int k = 0; k < AB; ++k) {
                            a_nx[k] = (wb + (unsigned)k * (unsigned)wstep)[a_off];
                            b_nx[k] = *reinterpret_cast<const Op*>(gk + b_byte);
                            gk += gstep * sizeof(T);
                        }
                    };
                    auto deal = [&]() {
#pragma unroll
                        for (int k = 0; k < AB; ++k) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);      // one MFMA
                            __builtin_amdgcn_sched_group_barrier(0x004, 12, 0);     // scalar address arithmetic
                            __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);      // vector
                            __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);      // two loads
                        }
                    };
                    if constexpr (!BREG) {
                        for (; k0 + 3 * AB <= kfast_end; k0 += 2 * AB) {
                            load_fast(a_s[1], b_s[1], k0 + AB);
#pragma unroll
                            for (int k = 0; k < AB; ++k) dd = GG::mma(a_s[0][k], b_s[0][k], dd);
                            deal();
                            load_fast(a_s[0], b_s[0], k0 + 2 * AB);
#pragma unroll
                            for (int k = 0; k < AB; ++k) dd = GG::mma(a_s[1][k], b_s[1][k], dd);
                            deal();
                        }
                    }
                    for (; k0 + AB < ksteps; k0 += 2 * AB) {
                        load_batch(a_s[1], b_s[1], wp, min(k0 + AB, k_last));
#pragma unroll
                        for (int k = 0; k < AB; ++k) dd = GG::mma(a_s[0][k], b_s[0][k], dd);
                        deal();
                        load_batch(a_s[0], b_s[0], wp, min(k0 + 2 * AB, k_last));
#pragma unroll
                        for (int k = 0; k < AB; ++k) dd = GG::mma(a_s[1][k], b_s[1][k], dd);
                        deal();
                    }
                    if (k0 < ksteps) {
#pragma unroll
                        for (int k = 0; k < AB; ++k) dd = GG::mma(a_s[0][k], b_s[0][k], dd);
                    }
                    return;
                }
                for (; k0 + AB < ksteps; k0 += 2 * AB) {
                    load_batch(a_s[1], b_s[1], wp, k0 + AB);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int k = 0; k < AB; ++k) dd = GG::mma(a_s[0][k], b_s[0][k], dd);
                    __builtin_amdgcn_sched_barrier(0);
                    if (k0 + 2 * AB < ksteps) load_batch(a_s[0], b_s[0], wp, k0 + 2 * AB);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int k = 0; k < AB; ++k) dd = GG::mma(a_s[1][k], b_s[1][k], dd);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (k0 < ksteps) {
#pragma unroll
                    for (int k = 0; k < AB; ++k) dd = GG::mma(a_s[0][k], b_s[0][k], dd);
                }
            };
            // register-resident operand: the batches of a pass past those that ride on the tap slots
            auto gemm_tail_reg = [&](typename MM::Acc& dd, const Op* wp) {
                if constexpr (BREG && BS > 1) {
                    Op a_x[2][AB];
                    if (NS * AB < ksteps) load_batch(a_x[0], nullptr, wp, NS * AB);
#pragma unroll
                    for (int kb = NS; kb < NS * BS; ++kb) {
                        if (kb * AB < ksteps) {
                            if ((kb + 1) * AB < ksteps && kb + 1 < NS * BS) load_batch(a_x[(kb + 1 - NS) & 1], nullptr, wp, (kb + 1) * AB);
#pragma unroll
                            for (int k = 0; k < AB; ++k) dd = GG::mma(a_x[(kb - NS) & 1][k], b_reg[kb * AB + k], dd);
                        }
                    }
                }
            };
            typename MM::Acc d_next = acc_zero<T>();
            if constexpr (BREG) {                                      // first pass: nothing to hide behind
#pragma unroll
                for (int ts = 0; ts < NS; ++ts) {
                    if (ts * AB < ksteps) {
                        Op a_cu[AB];
                        load_batch(a_cu, nullptr, wchunk, ts * AB);
#pragma unroll
                        for (int k = 0; k < AB; ++k) d_next = GG::mma(a_cu[k], b_reg[ts * AB + k], d_next);
                    }
                }
                gemm_tail_reg(d_next, wchunk);
            } else {
                gemm_tail(d_next, wchunk, 0);
            }
            // offsets and tap * dilation of the current and of the next tap slot, in two register sets
            // that swap roles from slot to slot (NS is even): copying "next" into "current" would have
            // to wait for the loads at the copy, a whole slot before the values are needed
            T o_buf[2][ND], kd_buf[2][ND];
            // grad_offset of an item that one workgroup owns alone: what the earlier chunks have written
            // for the slot's (tap, position) travels with the slot's offsets and the sum is stored --
            // plain loads and stores that stay in the L2 between two chunks, where float atomics are
            // limited to about one per clock and L2 channel (130 M of them per call on a 64-channel
            // 3x3x3 layer of 200 k positions)
            // (3-D kernels only: the short tap slots of the 2-D kernels lose more to the extra loads than
            // their few grad_offset elements cost in atomics, so the host asks for atomics there)
            constexpr bool RMW = COORD && ND == 3;
            T p_buf[2][ND];
            const bool rmw_prev = RMW && !goff_atomic && !first_chunk;        // uniform
            static_assert(NS % 2 == 0, "offset buffers alternate within a pass");
            // Kernel coordinates of this lane's tap in the next slot, counted up with the slots (the
            // taps of consecutive slots are TP / NS apart for every lane).  They live in registers: a
            // table in LDS would put a read into every slot that can only be waited for together with
            // the LDS adds issued behind it (LDS operations complete in order and the wait counter
            // cannot tell conditional adds apart), which serialises the adds with the next slot's
            // vector work.
            constexpr int STEP = TP / NS;
            static_assert(TP % NS == 0, "taps of consecutive slots are evenly spaced");
            int kq[ND];
            decode_tap<ND>(P, row_tap(0, q), kq);
            auto load_slot_offsets = [&](int tap_u, int ts) {         // tap_u: uniform tap of lane group 0 in slot ts
                T* o_nx = o_buf[ts & 1];
                T* kd_nx = kd_buf[ts & 1];
                const int tu = min(tap_u, P.kV - 1);
                const int dq = row_tap(ts * RPS, q) - row_tap(ts * RPS, 0);
                const int dqc = tu + dq < P.kV ? dq : 0;
                const unsigned lo = (unsigned)dqc * ND * P.outV + pos;
                const S* ob = off_dg + (size_t)tu * ND * P.outV;
#pragma unroll
                for (int a = 0; a < ND; ++a) o_nx[a] = Store<S>::ld((ob + (size_t)a * P.outV)[lo]);
                if constexpr (RMW) {
                    if (rmw_prev) {
                        const T* gb = goff_dg + (size_t)tu * ND * P.outV;
#pragma unroll
                        for (int a = 0; a < ND; ++a) p_buf[ts & 1][a] = (gb + (size_t)a * P.outV)[lo];
                    }
                }
#pragma unroll
                for (int a = 0; a < ND; ++a) kd_nx[a] = (T)(kq[a] * P.dil[slot<ND>(a)]);
#pragma unroll
                for (int st = 0; st < STEP; ++st) {                    // on to the next slot's tap: increment with carry
                    int carry = 1;
#pragma unroll
                    for (int a = ND - 1; a > 0; --a) {
                        kq[a] += carry;
                        carry = kq[a] >= P.k[slot<ND>(a)] ? 1 : 0;
                        kq[a] = carry ? 0 : kq[a];
                    }
                    kq[0] += carry;
                }
            };
            load_slot_offsets(row_tap(0, 0), 0);
            // grad_offset of a finished tap slot, held back until the loads of the next slot have been
            // issued: vector memory operations complete in order, so a load issued behind these
            // stores / atomics could only be waited for together with them
            bool pend = false;
            int pend_tap = 0;
            T pend_ga[ND];
#pragma unroll
            for (int a = 0; a < ND; ++a) pend_ga[a] = 0;
            auto write_goff = [&]() {
                if (pend) {
                    T* gp = goff_dg + (size_t)pend_tap * ND * P.outV + pos;
#pragma unroll
                    for (int a = 0; a < ND; ++a) {
                        if (goff_atomic) { if (pend_ga[a] != (T)0) atomic_add(gp + (size_t)a * P.outV, pend_ga[a]); }
                        else if (RMW || first_chunk) gp[(size_t)a * P.outV] = pend_ga[a];       // (3-D: the earlier chunks' sum is part of it)
                        else gp[(size_t)a * P.outV] += pend_ga[a];
                    }
                }
                pend = false;
            };
            // corner i of a sample sits at a fixed distance from its low corner (strides of the halo);
            // a corner that the reference collapses onto the low one carries weight zero instead
            unsigned coff[NC];
#pragma unroll
            for (int i = 0; i < NC; ++i)
                coff[i] = ND == 3 ? (unsigned)((((i >> 2) & 1) * he1 + ((i >> 1) & 1)) * he2 + (i & 1))
                                  : (unsigned)(((i >> 1) & 1) * he2 + (i & 1));

            for (int tap0 = 0; tap0 < P.kV; tap0 += TP) {
                const typename MM::Acc d = d_next;
                d_next = acc_zero<T>();
                const bool more = tap0 + TP < P.kV;                    // a pass follows: its MFMAs ride along
                int kz = 0;                                            // an opaque zero, for the same reason
                asm volatile("" : "+s"(kz));
                const Op* wnext = wchunk + (size_t)(tap0 / TP + 1) * wpass;
                if constexpr (!BREG) { if (more && ksteps > NS * AB) gemm_tail(d_next, wnext, NS * AB); }
                else { if (more) gemm_tail_reg(d_next, wnext); }
#pragma unroll
                for (int ts = 0; ts < NS; ++ts) {
                    // slots past the last tap (only in the last pass, which feeds no further MFMAs)
                    if (tap0 + row_tap(ts * RPS, 0) >= P.kV) continue;
                    const int tap = tap0 + row_tap(ts * RPS, q);
                    Op a_cu[AB], b_cu[AB];
                    const T* ofs = o_buf[ts & 1];
                    const T* kdf = kd_buf[ts & 1];
                    const bool do_mma = more && ts * AB < ksteps;      // uniform
                    // this slot's MFMA operands arrive while its geometry is set up; the offsets of the
                    // next tap slot travel while this one is worked on
                    if (do_mma) load_batch(a_cu, b_cu, wnext, ts * AB);
                    if (ts + 1 < NS) load_slot_offsets(tap0 + row_tap((ts + 1) * RPS, 0), ts + 1);
                    else load_slot_offsets(tap0 + TP + row_tap(0, 0), 0);
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (COORD) write_goff();
                    __builtin_amdgcn_sched_barrier(0);

                    // Geometry of this lane's (tap, position), following the reference sampler
                    // (deform3d/lib/deform_conv3d_cuda_kernel.cu:21-26,40-45,123-124) in a branch-free
                    // form: the coordinate is clamped into [0, size - 1]; low corner = floor, fraction
                    // toward the high corner = clamped coordinate - floor.  Where the reference collapses
                    // the high corner onto the low one (p <= 0, p >= size - 1) the fraction is 0, so the
                    // corner one step further carries weight 0 (a halo cell outside the volume holds 0)
                    // and every sample uses the same eight (four) cells at fixed strides.
                    const bool slot_ok = valid && tap < P.kV;
                    bool inside = slot_ok, inhalo = cells_ok;
                    bool intr[ND];                 // strictly between the collapse zones: the axis has a slope
                    T pq[ND], f[ND];
                    int u[ND];                     // low corner in halo coordinates
#pragma unroll
                    for (int a = 0; a < ND; ++a) {
                        const int s = slot<ND>(a);
                        const T top = (T)(P.in[s] - 1);
                        const T pa = (ibf[a] + kdf[a]) + ofs[a];
                        T pc;
                        if constexpr (sizeof(T) == 4) pc = __builtin_amdgcn_fmed3f(pa, 0.f, top);
                        else pc = fmin(fmax(pa, (T)0), top);
                        const T fl = floor(pc);
                        pq[a] = pa;
                        f[a] = pc - fl;
                        inside = inside && fabs(pa - pc) < (T)1;            // -1 < p < size, false for NaN
                        intr[a] = pa > (T)0 && pa < top;
                        u[a] = (int)fl - tg.hb[a];
                        inhalo = inhalo && (unsigned)u[a] < (unsigned)(H.hext[s] - 1);
                    }
                    {   // (mask arithmetic, no branch)
                        bool all_intr = true;
#pragma unroll
                        for (int a = 0; a < ND; ++a) all_intr = all_intr & intr[a];
                        inhalo = inhalo & (all_intr | !halo_nonfinite);
                    }
                    const bool near = inside && inhalo, far = inside && !inhalo;
                    unsigned base;
                    if constexpr (ND == 3) base = (unsigned)(__mul24(__mul24(u[0], he1) + u[1], he2) + u[2]);
                    else base = (unsigned)(__mul24(u[0], he2) + u[1]);
                    base = near ? base : 0u;       // lanes without a sample in the halo read cell 0 and add nothing
                    T cw[NC];
                    if constexpr (ND == 3) {       // multiplied in the reference's order (w_l * w_h * w_w)
                        const T fl = f[0], gl = (T)1 - fl, fh = f[1], gh = (T)1 - fh, fw = f[2], gw = (T)1 - fw;
                        const T a00 = gl * gh, a01 = gl * fh, a10 = fl * gh, a11 = fl * fh;
                        cw[0] = a00 * gw; cw[1] = a00 * fw; cw[2] = a01 * gw; cw[3] = a01 * fw;
                        cw[4] = a10 * gw; cw[5] = a10 * fw; cw[6] = a11 * gw; cw[7] = a11 * fw;
                    } else {
                        const T fh = f[0], gh = (T)1 - fh, fw = f[1], gw = (T)1 - fw;
                        cw[0] = gh * gw; cw[1] = gh * fw; cw[2] = fh * gw; cw[3] = fh * fw;
                    }
                    // grad-column values of this slot (rows past the chunk's channels: packed weights are
                    // zero there; the plain layout holds a neighbour's weights, so those are masked)
                    T gv[RPS];
#pragma unroll
                    for (int rr = 0; rr < RPS; ++rr) {
                        gv[rr] = d[ts * RPS + rr];
                        if constexpr (!PACKW) gv[rr] = row_ch(ts * RPS + rr, q) < nch ? gv[rr] : (T)0;
                    }
                    // Corner values of the input: one wide LDS read per corner for four of this lane's
                    // channels, issued by every lane, ahead of the MFMAs that cover their latency.
                    // d(sample)/d(coordinate) is linear in the corner values: it is applied once to
                    // the corner values weighted by gcol and summed over the lane's channels.  Every
                    // lane does this, outside any branch (a lane without a near sample works on cell
                    // 0 and drops the result): corner reads still pending at a branch that skips
                    // their use would make the compiler wait for the whole LDS queue, adds included,
                    // before the registers are written again.  Eight channels per slot go in two
                    // rounds of four (reads, half of the slot's MFMAs, sums) to bound the registers.
                    constexpr int RH = RPS > 4 ? RPS / 4 : 1, RW = RPS / RH;
                    T v[NC];
#pragma unroll
                    for (int h = 0; h < RH; ++h) {
                        T vv[NC][RW];
                        if constexpr (COORD) {
                            const T* ip = sIn + (size_t)base * CCH;
                            constexpr int GPV = swizzle_groups<T, CCH>();
                            if constexpr (GPV > 1) {
                                // the four-channel group read here sits at slot (group ^ voxel mod GPV) of its
                                // voxel (halo_stage_interleaved); the innermost halo extent is a multiple of GPV
                                // (host), so a corner's voxel is base + (i & 1) modulo GPV
                                static_assert(RW == 4, "a round reads one four-channel group");
                                const int grp = row_ch(ts * RPS + h * RW, q) / 4;
                                const T* ipx[2];
                                ipx[0] = ip + (((unsigned)grp ^ (base & (GPV - 1))) << 2);
                                ipx[1] = ip + (((unsigned)grp ^ ((base + 1) & (GPV - 1))) << 2);
#pragma unroll
                                for (int i = 0; i < NC; ++i)
#pragma unroll
                                    for (int rr = 0; rr < RW; ++rr) vv[i][rr] = ipx[i & 1][coff[i] * CCH + rr];
                            } else {
#pragma unroll
                                for (int i = 0; i < NC; ++i)
#pragma unroll
                                    for (int rr = 0; rr < RW; ++rr) vv[i][rr] = ip[coff[i] * CCH + row_ch(ts * RPS + h * RW + rr, q)];
                            }
                        }
                        // the next pass's MFMAs of this slot, in uniform control flow
                        if (do_mma) {
#pragma unroll
                            for (int k = h * (AB / RH); k < (h + 1) * (AB / RH); ++k)
                                d_next = GG::mma(a_cu[k], BREG ? b_reg[ts * AB + k] : b_cu[k], d_next);
                        }
                        if constexpr (COORD) {
#pragma unroll
                            for (int i = 0; i < NC; ++i) {
                                T acc_ = h == 0 ? gv[0] * vv[i][0] : v[i] + gv[h * RW] * vv[i][0];
#pragma unroll
                                for (int rr = 1; rr < RW; ++rr) acc_ += gv[h * RW + rr] * vv[i][rr];
                                v[i] = acc_;
                            }
                        }
                        if (h + 1 < RH) __builtin_amdgcn_sched_barrier(0);
                    }
                    T ga[ND];
#pragma unroll
                    for (int a = 0; a < ND; ++a) ga[a] = 0;
                    if constexpr (COORD) {
                        if constexpr (ND == 3) {
                            const T fl = f[0], gl = (T)1 - fl, fh = f[1], gh = (T)1 - fh, fw = f[2], gw = (T)1 - fw;
                            const T c00 = v[0] * gw + v[1] * fw, c01 = v[2] * gw + v[3] * fw;
                            const T c10 = v[4] * gw + v[5] * fw, c11 = v[6] * gw + v[7] * fw;
                            const T dl = (c10 - c00) * gh + (c11 - c01) * fh;
                            const T dh = (c01 - c00) * gl + (c11 - c10) * fl;
                            const T dw = ((v[1] - v[0]) * gh + (v[3] - v[2]) * fh) * gl +
                                         ((v[5] - v[4]) * gh + (v[7] - v[6]) * fh) * fl;
                            ga[0] = (near && intr[0]) ? dl : (T)0; ga[1] = (near && intr[1]) ? dh : (T)0;
                            ga[2] = (near && intr[2]) ? dw : (T)0;
                        } else {
                            const T fh = f[0], gh = (T)1 - fh, fw = f[1], gw = (T)1 - fw;
                            const T dh = (v[2] - v[0]) * gw + (v[3] - v[1]) * fw;
                            const T dw = (v[1] - v[0]) * gh + (v[3] - v[2]) * fh;
                            ga[0] = (near && intr[0]) ? dh : (T)0; ga[1] = (near && intr[1]) ? dw : (T)0;
                        }
                    }
                    if (near) {
                        Cell* cp = sG + base;
                        if constexpr (PAIR) {
#pragma unroll
                            for (int rr = 0; rr < RPS; rr += 2) {          // consecutive registers hold consecutive channels
                                const float g0 = (float)gv[rr] * scale32, g1 = (float)gv[rr + 1] * scale32;
                                const int pl = row_ch(ts * RPS + rr, q) / 2;
#pragma unroll
                                for (int i = 0; i < NC; ++i) LdsCell<float>::add2(cp + coff[i] + pl * hs, (float)cw[i], g0, g1);
                            }
                        } else {
#pragma unroll
                            for (int rr = 0; rr < RPS; ++rr) {
                                const double gs = LdsCell<T>::pre(gv[rr], scale);
                                const int cl = row_ch(ts * RPS + rr, q);
#pragma unroll
                                for (int i = 0; i < NC; ++i) LdsCell<T>::add(cp + coff[i] + cl * hs, (double)cw[i], gs);
                            }
                        }
                    }
                    if constexpr (COORD && ND == 3) {
                        // out-of-range samples of the 3-D operator: -|gcol| per axis with p <= -1, +|gcol|
                        // with p >= the LENGTH extent (h and w are compared with it too), summed over the
                        // channels (deform3d/lib/deform_conv3d_cuda_kernel.cu:470-481).  Selected, not
                        // multiplied: 0 * inf would be NaN where the reference adds nothing
                        const bool oor = slot_ok && !inside && !P.oob_zero;
                        if (__any(oor)) {
                            T asum = 0;
#pragma unroll
                            for (int rr = 0; rr < RPS; ++rr) asum += fabs(gv[rr]);
                            if (oor) {
#pragma unroll
                                for (int a = 0; a < ND; ++a)
                                    ga[a] = pq[a] <= (T)-1 ? -asum : (pq[a] >= (T)P.in[0] ? asum : (T)0);
                            }
                        }
                    }
                    if (__any(far)) {              // rare: samples that reach past the halo go to global memory
                        TapGeo<T, ND> t;           // the reference's corner rule on the same coordinate
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
                        T fcw[NC];
                        if constexpr (ND == 3) {
                            const T fl = t.f[0], gl = (T)1 - fl, fh = t.f[1], gh = (T)1 - fh, fw = t.f[2], gw = (T)1 - fw;
                            fcw[0] = gl * gh * gw; fcw[1] = gl * gh * fw; fcw[2] = gl * fh * gw; fcw[3] = gl * fh * fw;
                            fcw[4] = fl * gh * gw; fcw[5] = fl * gh * fw; fcw[6] = fl * fh * gw; fcw[7] = fl * fh * fw;
                        } else {
                            const T fh = t.f[0], gh = (T)1 - fh, fw = t.f[1], gw = (T)1 - fw;
                            fcw[0] = gh * gw; fcw[1] = gh * fw; fcw[2] = fh * gw; fcw[3] = fh * fw;
                        }
#pragma unroll
                        for (int rr = 0; rr < RPS; ++rr) {
                            const int cl = row_ch(ts * RPS + rr, q);
                            if (far && cl < nch) {
                                const T g1 = gv[rr];
                                const size_t chan = ((size_t)n * P.C_in + cc0 + cl + kz) * P.inV;
                                T* gc = gin + chan;
#pragma unroll
                                for (int i = 0; i < NC; ++i) atomic_add(gc + t.idx[i], fcw[i] * g1);
                                if constexpr (COORD) {
                                    const S* ic = in + chan;
                                    T v[NC];
#pragma unroll
                                    for (int i = 0; i < NC; ++i) v[i] = g1 * Store<S>::ld(ic[t.idx[i]]);
                                    if constexpr (ND == 3) {
                                        const T fl = t.f[0], gl = (T)1 - fl, fh = t.f[1], gh = (T)1 - fh, fw = t.f[2], gw = (T)1 - fw;
                                        const T c00 = v[0] * gw + v[1] * fw, c01 = v[2] * gw + v[3] * fw;
                                        const T c10 = v[4] * gw + v[5] * fw, c11 = v[6] * gw + v[7] * fw;
                                        ga[0] += (c10 - c00) * gh + (c11 - c01) * fh;
                                        ga[1] += (c01 - c00) * gl + (c11 - c10) * fl;
                                        ga[2] += ((v[1] - v[0]) * gh + (v[3] - v[2]) * fh) * gl +
                                                 ((v[5] - v[4]) * gh + (v[7] - v[6]) * fh) * fl;
                                    } else {
                                        const T fh = t.f[0], gh = (T)1 - fh, fw = t.f[1], gw = (T)1 - fw;
                                        ga[0] += (v[2] - v[0]) * gw + (v[3] - v[1]) * fw;
                                        ga[1] += (v[1] - v[0]) * gh + (v[3] - v[2]) * fh;
                                    }
                                }
                            }
                        }
                    }
                    if constexpr (COORD) {
                        // channels of one (tap, position) that sit in other lane groups are summed in
                        if constexpr (RPS < CCH) {
#pragma unroll
                            for (int a = 0; a < ND; ++a)
#pragma unroll
                                for (int sh = TN; sh < TN * (CCH / RPS); sh <<= 1) ga[a] += __shfl_xor(ga[a], sh);
                        }
                        // written at the start of the next slot, behind that slot's loads (see write_goff)
                        const bool owner = (RPS == CCH) || (q % (CCH / RPS)) == 0;
                        pend = slot_ok && owner;
                        pend_tap = tap;
#pragma unroll
                        for (int a = 0; a < ND; ++a) {
                            if constexpr (RMW) pend_ga[a] = rmw_prev ? ga[a] + p_buf[ts & 1][a] : ga[a];
                            else pend_ga[a] = ga[a];
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);      // one tap slot at a time: keeps the live register set small
                }
            }
            if constexpr (COORD) write_goff();
            first_chunk = false;
            __syncthreads();                        // all LDS adds of this chunk have landed
            for (int v = threadIdx.x; v < H.hvol; v += WGS) {
                const unsigned gv = sTab[v];
                if (gv == ~0u) continue;            // halo cell outside the volume: never touched
                if constexpr (PAIR) {
                    for (int c = 0; c < nch; c += 2) {
                        const Cell cell = sG[(c / 2) * hs + v];
                        if (cell != (Cell)0) {
                            float v0, v1;
                            LdsCell<float>::value2(cell, inv_scale, v0, v1);
                            T* gp = gin + ((size_t)n * P.C_in + cc0 + c) * P.inV + gv;
                            if (v0 != 0.f) atomic_add(gp, (T)v0);
                            if (c + 1 < nch && v1 != 0.f) atomic_add(gp + P.inV, (T)v1);
                        }
                    }
                } else {
                    for (int c = 0; c < nch; ++c) {
                        const Cell cell = sG[c * hs + v];
                        if (cell != (Cell)0)
                            atomic_add(gin + ((size_t)n * P.C_in + cc0 + c) * P.inV + gv, (T)LdsCell<T>::value(cell, inv_scale));
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Backward to weight: gW[g*M+m][cl][tap] += sum_{n,pos} gout[n][g*M+m][pos] * sample(in[n][g*Cg+cl], tap, pos)
// replaces the second deformable_im2col + Sgemm(beta=1) of deform3d/lib/deform_conv3d_cuda.cpp:283-320.
// The reduction runs over positions, so both MFMA operands want lanes along the non-reduced
// dimension: A[m][pos] and B[pos][channel].  With the input and grad_output held channels-last
// ([voxel][channel], [position][out channel]) both operands are contiguous across the lanes of a
// lane group: lane (j, q) samples channel c0 + j at position 2*ks + q of the slab (8 or 4
// coalesced corner loads) and loads grad_output row m_base + j of the same position.  The
// geometry of the slab's TN positions is computed once by the position-owning lanes and handed
// to the channel lanes through a wavefront-private LDS record.
// A workgroup keeps one (tap, channel tile, m chunk) for its whole life; its wavefronts stride
// over position slabs independently (no workgroup barriers), so the [MT*TN x TN] accumulator
// stays in registers; each workgroup writes one partial tile per split and a small second kernel
// sums the splits into grad_weight (deterministic, no atomics).
// dynamic LDS = WAVES * TN * (TN+1) * sizeof(T).
template <typename T, int ND, int MT>
__global__ __launch_bounds__(WG) void backward_weight_kernel(Params P, const T* __restrict__ in_cl,
                                                             const T* __restrict__ off,
                                                             const T* __restrict__ gout_cl, T* __restrict__ partial) {
    using MM = Mma<T>;
    constexpr int TN = MM::TN, KL = MM::KL, NC = 1 << ND;
    // geometry record of a (tap, position), written once per slab and read by every reduction step
    __shared__ __align__(16) unsigned sIdx[WAVES][TN][NC];   // byte offset of each corner's channel 0 inside the sample, 0 when the sample is dead
    __shared__ __align__(16) T sCw[WAVES][TN][NC];           // interpolation weight of each corner, 0 when the sample is dead
    __shared__ unsigned sLive[WAVES][TN];                    // 1 when the sample is live
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* sAcc = reinterpret_cast<T*>(smem_raw);                // [WAVES][TN][TN + 1]: the wavefronts' partial tiles, one row tile at a time
    // (the wavefront number as a scalar: the slab, the sample and the operand bases derived from it
    // then live in scalar registers and the loads take the scalar-base + 32-bit-offset form)
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane % TN, q = lane / TN;

    // 1-D grid of nctiles * mchunks * nsplit * kV workgroups in an XCD-contiguous order with the tap
    // fastest: the workgroups that gather around the same positions and channels share an L2
    const unsigned wg = xcd_contiguous(blockIdx.x, gridDim.x);
    const int tap = wg % (unsigned)P.kV;
    const int split = (wg / (unsigned)P.kV) % (unsigned)P.nsplit;
    const unsigned zz = (wg / (unsigned)P.kV) / (unsigned)P.nsplit;
    const int mchunk = zz % P.mchunks;
    int z = zz / P.mchunks;
    // locate channel tile z: segments are the intersections of convolution groups with deformable groups
    int g = 0, dg = 0, c0 = 0, ce = 0;
    bool found = false;
    for (g = 0; g < P.G && !found; ++g) {
        const int cg0 = g * P.Cg, cg1 = cg0 + P.Cg;
        for (dg = cg0 / P.cpg; dg <= (cg1 - 1) / P.cpg; ++dg) {
            const int cb = max(cg0, dg * P.cpg);
            ce = min(cg1, (dg + 1) * P.cpg);
            const int nt = (ce - cb + TN - 1) / TN;
            if (z < nt) { c0 = cb + z * TN; found = true; break; }
            z -= nt;
        }
        if (found) break;
    }
    if (!found) return;     // uniform for the workgroup

    int kk[ND], kd[ND];
    decode_tap<ND>(P, tap, kk);
#pragma unroll
    for (int a = 0; a < ND; ++a) kd[a] = kk[a] * P.dil[slot<ND>(a)];

    typename MM::Acc acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = acc_zero<T>();

    const int m_base = mchunk * MT * TN;
    const unsigned cj = (unsigned)min(c0 + j, P.C_in - 1);          // clamped: dead lanes still load legally
    // operands are addressed by 32-bit byte offsets from the sample's base (the host checks that a
    // sample of either tensor stays below 4 GiB)
    const unsigned cjB = cj * (unsigned)sizeof(T);
    const unsigned cinB = (unsigned)P.C_in * (unsigned)sizeof(T), rowB = (unsigned)P.C_out * (unsigned)sizeof(T);
    unsigned mrowB[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = m_base + mt * TN + j;
        mrowB[mt] = (unsigned)(g * P.M + min(m, P.M - 1)) * (unsigned)sizeof(T);
    }

    const int slabs_per_sample = (P.outV + TN - 1) / TN;
    const int nslabs = P.N * slabs_per_sample;
    for (int slab = split * WAVES + wave; slab < nslabs; slab += P.nsplit * WAVES) {
        const int n = slab / slabs_per_sample;
        const unsigned p0 = (unsigned)(slab % slabs_per_sample) * TN;
        const unsigned pos = p0 + j;
        const bool valid = pos < P.outV;
        const unsigned posc = valid ? pos : P.outV - 1;
        int o[ND], ib[ND];
        decode_pos<ND>(P, posc, o);
#pragma unroll
        for (int a = 0; a < ND; ++a) ib[a] = o[a] * P.stride[slot<ND>(a)] - P.pad[slot<ND>(a)];
        TapGeo<T, ND> t;
        {
            T offv[ND];
            load_offsets<T, ND>(P, off + (((size_t)n * P.DG + dg) * P.kV + tap) * ND * P.outV, posc, offv);
            tap_setup_noidx<T, ND>(P, offv, ib, kd, t);
        }
        const bool live = valid && t.inside;

        // LDS operations of one wavefront execute in order; the fences only pin the compiler
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (q == 0) {
            T cw[NC];                              // multiplied in the reference's order (w_l * w_h * w_w)
            if constexpr (ND == 3) {
                const T fl = t.f[0], gl = (T)1 - fl, fh = t.f[1], gh = (T)1 - fh, fw = t.f[2], gw = (T)1 - fw;
                cw[0] = gl * gh * gw; cw[1] = gl * gh * fw; cw[2] = gl * fh * gw; cw[3] = gl * fh * fw;
                cw[4] = fl * gh * gw; cw[5] = fl * gh * fw; cw[6] = fl * fh * gw; cw[7] = fl * fh * fw;
            } else {
                const T fh = t.f[0], gh = (T)1 - fh, fw = t.f[1], gw = (T)1 - fw;
                cw[0] = gh * gw; cw[1] = gh * fw; cw[2] = fh * gw; cw[3] = fh * fw;
            }
            unsigned cb[NC];
            tap_corner_offsets<T, ND>(P, t, live, cinB, cb);
#pragma unroll
            for (int i = 0; i < NC; ++i) sIdx[wave][j][i] = cb[i];
#pragma unroll
            for (int i = 0; i < NC; ++i) sCw[wave][j][i] = live ? cw[i] : (T)0;
            sLive[wave][j] = live ? 1u : 0u;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        const char* in_n = reinterpret_cast<const char*>(in_cl + (size_t)n * P.inV * P.C_in);        // scalar bases
        const char* go_n = reinterpret_cast<const char*>(gout_cl + (size_t)n * P.outV * P.C_out);
        const unsigned a_first = (p0 + (unsigned)q) * rowB;          // grad_output row of this lane's position in step 0
        const unsigned a_last = (P.outV - 1) * rowB;                 // positions past the end re-read the last row (masked below)
        // reduction over the slab's positions, software pipelined: while step ks is interpolated and
        // multiplied, the geometry record, the corner values and the grad_output rows of step ks + 1
        // are already in flight
        constexpr int NK = TN / KL;
        constexpr int DEPTH = 1;                    // steps in flight ahead of the one being multiplied (2 is no faster)
        T cn[DEPTH][NC], an[DEPTH][MT], wn[DEPTH][NC];
        bool lvn[DEPTH];
        auto fetch = [&](int ks, int slot_) {
            const int pp = ks * KL + q;             // position of the slab this lane group works on
            unsigned ix[NC];
#pragma unroll
            for (int i = 0; i < NC; ++i) ix[i] = sIdx[wave][pp][i];
#pragma unroll
            for (int i = 0; i < NC; ++i) wn[slot_][i] = sCw[wave][pp][i];
            lvn[slot_] = sLive[wave][pp] != 0u;
            const unsigned ao = min(a_first + (unsigned)(ks * KL) * rowB, a_last);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)         // A[row = m][k = position]; legal for every lane
                an[slot_][mt] = *reinterpret_cast<const T*>(go_n + (ao + mrowB[mt]));
#pragma unroll
            for (int i = 0; i < NC; ++i)            // dead samples read voxel 0
                cn[slot_][i] = *reinterpret_cast<const T*>(in_n + (ix[i] + cjB));
        };
#pragma unroll
        for (int d0 = 0; d0 < DEPTH; ++d0) fetch(d0, d0);
#pragma unroll
        for (int ks = 0; ks < NK; ++ks) {
            const int sl = ks % DEPTH;
            T cc[NC], ac[MT], wc[NC];
#pragma unroll
            for (int i = 0; i < NC; ++i) cc[i] = cn[sl][i];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) ac[mt] = an[sl][mt];
#pragma unroll
            for (int i = 0; i < NC; ++i) wc[i] = wn[sl][i];
            const bool lvc = lvn[sl];
            if (ks + DEPTH < NK) fetch(ks + DEPTH, sl);
            __builtin_amdgcn_sched_barrier(0);      // later steps' loads are issued before this step's arithmetic
            T v = wc[0] * cc[0];                    // weighted corner sum, as the reference's sampler forms it
#pragma unroll
            for (int i = 1; i < NC; ++i) v += wc[i] * cc[i];
            // B[k = position][col = channel j], exactly zero for a dead sample and for a position past
            // the end.  Nothing else is masked: a row of A only reaches its own row of the tile and a
            // column of B its own column, and rows past M / columns past the segment are not stored.
            const T b = lvc ? v : (T)0;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[mt] = MM::mma(ac[mt], b, acc[mt]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // One row tile at a time, so that the LDS footprint (and with it the number of resident
    // workgroups that hide the gather latency) does not grow with MT.
    constexpr int LDA = TN + 1;
    T* pt = partial + ((size_t)split * P.kV + tap) * P.C_out * P.Cg;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        if (mt) __syncthreads();                    // readers of the previous tile are done
#pragma unroll
        for (int r = 0; r < MM::NACC; ++r) sAcc[((size_t)wave * TN + MM::row(r, q)) * LDA + j] = acc[mt][r];
        __syncthreads();
        for (int e = threadIdx.x; e < TN * TN; e += WG) {
            const int mr = e / TN, cc = e % TN;
            const int m = m_base + mt * TN + mr, c = c0 + cc;
            if (m < P.M && c < ce) {
                T sum = 0;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) sum += sAcc[((size_t)w * TN + mr) * LDA + cc];
                pt[((size_t)g * P.M + m) * P.Cg + (c - g * P.Cg)] = sum;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Backward to weight with 16-bit storage (S = Bf16 / Fp16, float arithmetic): the same
// decomposition as backward_weight_kernel -- a workgroup keeps one (tap, channel tile, m chunk),
// its wavefronts stride over slabs of TN positions, one partial tile per split -- on the 16-bit
// matrix instructions v_mfma_f32_32x32x8_bf16 / _f16 (float accumulation).  One instruction reduces
// over 8 positions: lane (j, q) supplies the positions 8 * step + 4 * q + 0..3 of its row / column.
//  * B operand (sampled columns): the input is held channels-last in its storage format and a lane
//    fetches TWO neighbouring channels of a corner with one 4-byte load, so a channel tile is 64
//    channels wide (columns j of two accumulator tiles: channels first + 2 j and first + 2 j + 1) and
//    a sample costs half the load instructions of the float kernel; interpolation in float, the
//    sampled values rounded to the storage format for the matrix instruction (as the forward pass
//    does).  The host calls this kernel only for an even number of input channels with even
//    segment starts (4-byte alignment of the channel pairs).
//  * A operand: grad_output channels-last in its storage format ([n][position][output channel]): the
//    lanes of a load read consecutive output channels of one position (in grad_output's own layout
//    every lane of a load would touch a cache line of its own).
// dynamic LDS = WAVES * TN * (TN + 1) * 4 bytes, as in the float kernel.
template <int ND, int MT, typename S>
__global__ __launch_bounds__(WG) void backward_weight16_kernel(Params P, const S* __restrict__ in_cl, const S* __restrict__ off,
                                                               const S* __restrict__ gout_cl, float* __restrict__ partial) {
    typedef float T;
    using MM = Mma<float>;
    constexpr int TN = MM::TN, NC = 1 << ND, CT = 2 * TN;          // CT channels per tile
    __shared__ __align__(16) unsigned sIdx[WAVES][TN][NC];   // byte offset of each corner's channel 0 inside the sample, 0 when the sample is dead
    __shared__ __align__(16) T sCw[WAVES][TN][NC];           // interpolation weight of each corner, 0 when the sample is dead
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* sAcc = reinterpret_cast<T*>(smem_raw);                // [WAVES][TN][TN + 1]
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane % TN, q = lane / TN;

    const unsigned wg = xcd_contiguous(blockIdx.x, gridDim.x);
    const int tap = wg % (unsigned)P.kV;
    const int split = (wg / (unsigned)P.kV) % (unsigned)P.nsplit;
    const unsigned zz = (wg / (unsigned)P.kV) / (unsigned)P.nsplit;
    const int mchunk = zz % P.mchunks;
    int z = zz / P.mchunks;
    int g = 0, dg = 0, c0 = 0, ce = 0;
    bool found = false;
    for (g = 0; g < P.G && !found; ++g) {
        const int cg0 = g * P.Cg, cg1 = cg0 + P.Cg;
        for (dg = cg0 / P.cpg; dg <= (cg1 - 1) / P.cpg; ++dg) {
            const int cb = max(cg0, dg * P.cpg);
            ce = min(cg1, (dg + 1) * P.cpg);
            const int nt = (ce - cb + CT - 1) / CT;
            if (z < nt) { c0 = cb + z * CT; found = true; break; }
            z -= nt;
        }
        if (found) break;
    }
    if (!found) return;     // uniform for the workgroup

    int kk[ND], kd[ND];
    decode_tap<ND>(P, tap, kk);
#pragma unroll
    for (int a = 0; a < ND; ++a) kd[a] = kk[a] * P.dil[slot<ND>(a)];

    typename MM::Acc acc[2][MT];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[t][mt] = acc_zero<T>();

    const int m_base = mchunk * MT * TN;
    // this lane's channel pair (clamped to the last whole pair of the tensor: dead lanes still load legally)
    const unsigned cjB = (unsigned)min(c0 + 2 * j, P.C_in - 2) * (unsigned)sizeof(S);
    const unsigned cinB = (unsigned)P.C_in * (unsigned)sizeof(S);
    unsigned mrow[MT];                              // this lane's output channel (clamped: rows past M are not stored)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) mrow[mt] = (unsigned)(g * P.M + min(m_base + mt * TN + j, P.M - 1));

    const int slabs_per_sample = (P.outV + TN - 1) / TN;
    const int nslabs = P.N * slabs_per_sample;
    for (int slab = split * WAVES + wave; slab < nslabs; slab += P.nsplit * WAVES) {
        const int n = slab / slabs_per_sample;
        const unsigned p0 = (unsigned)(slab % slabs_per_sample) * TN;
        const unsigned pos = p0 + j;
        const bool valid = pos < P.outV;
        const unsigned posc = valid ? pos : P.outV - 1;
        int o[ND], ib[ND];
        decode_pos<ND>(P, posc, o);
#pragma unroll
        for (int a = 0; a < ND; ++a) ib[a] = o[a] * P.stride[slot<ND>(a)] - P.pad[slot<ND>(a)];
        TapGeo<T, ND> t;
        {
            const S* op = off + (((size_t)n * P.DG + dg) * P.kV + tap) * ND * P.outV;
            T offv[ND];
#pragma unroll
            for (int a = 0; a < ND; ++a) offv[a] = Store<S>::ld(op[(size_t)a * P.outV + posc]);
            tap_setup_noidx<T, ND>(P, offv, ib, kd, t);
        }
        const bool live = valid && t.inside;

        // LDS operations of one wavefront execute in order; the fences only pin the compiler
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (q == 0) {
            T cw[NC];                              // multiplied in the reference's order (w_l * w_h * w_w)
            if constexpr (ND == 3) {
                const T fl = t.f[0], gl = (T)1 - fl, fh = t.f[1], gh = (T)1 - fh, fw = t.f[2], gw = (T)1 - fw;
                cw[0] = gl * gh * gw; cw[1] = gl * gh * fw; cw[2] = gl * fh * gw; cw[3] = gl * fh * fw;
                cw[4] = fl * gh * gw; cw[5] = fl * gh * fw; cw[6] = fl * fh * gw; cw[7] = fl * fh * fw;
            } else {
                const T fh = t.f[0], gh = (T)1 - fh, fw = t.f[1], gw = (T)1 - fw;
                cw[0] = gh * gw; cw[1] = gh * fw; cw[2] = fh * gw; cw[3] = fh * fw;
            }
            unsigned cb[NC];
            tap_corner_offsets<T, ND>(P, t, live, cinB, cb);
#pragma unroll
            for (int i = 0; i < NC; ++i) sIdx[wave][j][i] = cb[i];
#pragma unroll
            for (int i = 0; i < NC; ++i) sCw[wave][j][i] = live ? cw[i] : (T)0;      // a dead sample weighs nothing
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        const char* in_n = reinterpret_cast<const char*>(in_cl + (size_t)n * P.inV * P.C_in);        // scalar bases
        const S* go_n = gout_cl + (size_t)n * P.C_out * P.outV;
        constexpr int NK = TN / 8;                  // matrix instructions (reduction steps of 8 positions) per slab
        // Software pipeline over the TN / 2 (position, lane group) units of the slab with the corner
        // pairs of four units in flight (a ring of four register sets: unit u is interpolated from set
        // u % 4, which then takes the loads of unit u + 4); every fourth unit completes a reduction
        // step, whose grad_output rows were requested a step earlier.
        constexpr int RING = 4;
        unsigned cn[RING][NC];
        typename Mma16<S>::Vec an[MT];
        auto fetch_corners = [&](int u) {           // unit u: position 8 * (u / 4) + 4 * q + u % 4 of the slab
            const int pp = (u / 4) * 8 + 4 * q + (u % 4);
            unsigned ix[NC];
#pragma unroll
            for (int i = 0; i < NC; ++i) ix[i] = sIdx[wave][pp][i];
#pragma unroll
            for (int i = 0; i < NC; ++i) cn[u % RING][i] = *reinterpret_cast<const unsigned*>(in_n + (ix[i] + cjB));      // two channels
        };
        auto fetch_rows = [&](int ks) {             // A[row = m][k = position]: four consecutive positions, clamped at the end of the sample
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                S a4[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) a4[r] = go_n[min(p0 + (unsigned)(ks * 8 + 4 * q + r), P.outV - 1) * (unsigned)P.C_out + mrow[mt]];
                an[mt] = __builtin_bit_cast(typename Mma16<S>::Vec, a4);
            }
        };
        fetch_rows(0);
#pragma unroll
        for (int u = 0; u < RING; ++u) fetch_corners(u);
        float ve[4], vo[4];                         // even / odd channel of the pair at the step's four positions
#pragma unroll
        for (int u = 0; u < NK * 4; ++u) {
            unsigned cc[NC];
            T wc[NC];
#pragma unroll
            for (int i = 0; i < NC; ++i) cc[i] = cn[u % RING][i];
            {
                const int pp = (u / 4) * 8 + 4 * q + (u % 4);
#pragma unroll
                for (int i = 0; i < NC; ++i) wc[i] = sCw[wave][pp][i];
            }
            typename Mma16<S>::Vec ac[MT];
            if (u % 4 == 3) {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) ac[mt] = an[mt];
                if (u / 4 + 1 < NK) fetch_rows(u / 4 + 1);
            }
            __builtin_amdgcn_sched_barrier(0);
            float se = 0.f, so = 0.f;
#pragma unroll
            for (int i = 0; i < NC; ++i) {
                const unsigned short lb = (unsigned short)(cc[i] & 0xffffu), hb = (unsigned short)(cc[i] >> 16);
                se += wc[i] * Store<S>::ld(__builtin_bit_cast(S, lb));
                so += wc[i] * Store<S>::ld(__builtin_bit_cast(S, hb));
            }
            // (dead samples and positions past the end carry weight zero; an input value that is not
            // finite there gives NaN, as 0 * inf does in the reference's GEMM on its zero column rows)
            ve[u % 4] = se;
            vo[u % 4] = so;
            if (u + RING < NK * 4) fetch_corners(u + RING);       // into the set just consumed
            if (u % 4 == 3) {
                const typename Mma16<S>::Vec be = Mma16<S>::pack(ve), bo = Mma16<S>::pack(vo);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    acc[0][mt] = Mma16<S>::mma(ac[mt], be, acc[0][mt]);
                    acc[1][mt] = Mma16<S>::mma(ac[mt], bo, acc[1][mt]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    constexpr int LDA = TN + 1;
    T* pt = partial + ((size_t)split * P.kV + tap) * P.C_out * P.Cg;
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            __syncthreads();                        // readers of the previous tile are done
#pragma unroll
            for (int r = 0; r < MM::NACC; ++r) sAcc[((size_t)wave * TN + MM::row(r, q)) * LDA + j] = acc[t2][mt][r];
            __syncthreads();
            for (int e = threadIdx.x; e < TN * TN; e += WG) {
                const int mr = e / TN, cc = e % TN;
                const int m = m_base + mt * TN + mr, c = c0 + 2 * cc + t2;
                if (m < P.M && c < ce) {
                    T sum = 0;
#pragma unroll
                    for (int w = 0; w < WAVES; ++w) sum += sAcc[((size_t)w * TN + mr) * LDA + cc];
                    pt[((size_t)g * P.M + m) * P.Cg + (c - g * P.Cg)] = sum;
                }
            }
        }
}

// grad_weight[g*M+m][cl][tap] += sum over splits of partial[split][tap][g*M+m][cl]
// 256 threads = 64 consecutive elements x 4 lanes of splits: lane l adds the splits l, l + 4, ...
// (loads of a lane independent of each other), then the four sums are added in the order of l, so
// the result does not depend on timing.
template <typename T>
__global__ __launch_bounds__(256) void reduce_weight_partials_kernel(const T* __restrict__ partial, T* __restrict__ gw, int nsplit, int kV,
                                                                     size_t rows_x_cg /* C_out * Cg */) {
    __shared__ T part[4][64];
    const size_t total = (size_t)kV * rows_x_cg;
    const int e = threadIdx.x & 63, l = threadIdx.x >> 6;
    for (size_t i0 = (size_t)blockIdx.x * 64; i0 < total; i0 += (size_t)gridDim.x * 64) {
        const size_t i = i0 + e;
        T sum = 0;
        if (i < total) {
            const T* p = partial + i;
            int s = l;
            for (; s + 12 < nsplit; s += 16) {
                const T a = p[(size_t)s * total], b = p[(size_t)(s + 4) * total], c = p[(size_t)(s + 8) * total], d = p[(size_t)(s + 12) * total];
                sum += a; sum += b; sum += c; sum += d;
            }
            for (; s < nsplit; s += 4) sum += p[(size_t)s * total];
        }
        part[l][e] = sum;
        __syncthreads();
        if (l == 0 && i < total) {
            const size_t tap = i / rows_x_cg, rc = i % rows_x_cg;     // rc = (g*M + m) * Cg + cl
            gw[rc * kV + tap] += ((part[0][e] + part[1][e]) + part[2][e]) + part[3][e];
        }
        __syncthreads();
    }
}

// Both layout changes of backward_weight in one launch: z < N copies tensor A, z >= N tensor B
// (grid: the larger of the two extents along x and y, 2 * N along z).
template <typename T>
__global__ void to_channels_last_pair_kernel(const T* __restrict__ srcA, T* __restrict__ dstA, int CA, unsigned VA,
                                             const T* __restrict__ srcB, T* __restrict__ dstB, int CB, unsigned VB, int N) {
    __shared__ T tile[32][33];
    const bool second = (int)blockIdx.z >= N;
    const T* src = second ? srcB : srcA;
    T* dst = second ? dstB : dstA;
    const int C = second ? CB : CA;
    const unsigned V = second ? VB : VA;
    const unsigned v0 = blockIdx.x * 32;
    const int c0 = blockIdx.y * 32;
    if (v0 >= V || c0 >= C) return;                 // uniform for the block
    const size_t base = (size_t)(second ? blockIdx.z - N : blockIdx.z) * C * V;
    for (int i = threadIdx.y; i < 32; i += 8) {
        const int c = c0 + i;
        const unsigned v = v0 + threadIdx.x;
        if (c < C && v < V) tile[i][threadIdx.x] = src[base + (size_t)c * V + v];
    }
    __syncthreads();
    for (int i = threadIdx.y; i < 32; i += 8) {
        const unsigned v = v0 + i;
        const int c = c0 + threadIdx.x;
        if (c < C && v < V) dst[base + (size_t)v * C + c] = tile[threadIdx.x][i];
    }
}

}  // namespace dcn
