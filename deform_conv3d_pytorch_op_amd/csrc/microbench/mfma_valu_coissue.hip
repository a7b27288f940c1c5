// Which vector instructions run alongside MFMA on gfx950?  For each pair: the MFMA stream alone, the
// vector stream alone, and both in the same wavefronts; "overlap" is how much of the shorter stream the
// combination hides (0 %: the times add).  Instruction mixes are pinned with inline asm; registers only,
// no memory traffic.  Build and run (no arguments):
//   hipcc --offload-arch=gfx950 -O3 -Xclang -target-feature -Xclang -packed-fp32-ops -o mfma_valu_coissue mfma_valu_coissue.hip
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1); } } while (0)
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef double d4v __attribute__((ext_vector_type(4)));

// VK: 0 v_fma_f32, 1 v_add_u32, 2 v_cndmask_b32, 3 v_fma_f64, 4 v_cvt_f64_f32, 5 v_mul_f32, 6 v_lshl_add_u32, 7 v_cmp_lt_f32, 8 v_add_f32, 9 v_cvt_i32_f32, 10 v_mad_u32_u24, 11 v_med3_f32, 12 v_floor_f32
// MK: 0 none, 1 32x32x2 f32, 2 16x16x4 f32, 3 16x16x4 f64, 4 32x32x8 bf16, 5 32x32x16 bf16 (both accumulate in float),
//     6 32x32x16 bf16 with the accumulator in AGPRs, 7 32x32x2 f32 with the accumulator in AGPRs
template <int MK, int NM, int VK, int NV, int NT>
__global__ __launch_bounds__(NT) void k(int iters, float* out) {
    f16v acc0 = {0}, acc1 = {0};
    f4v b0 = {0, 0, 0, 0}, b1 = {0, 0, 0, 0};
    d4v c0 = {0, 0, 0, 0}, c1 = {0, 0, 0, 0};
    float a = threadIdx.x * 1e-3f, b = 1.0001f;
    double ad = a, bd = b;
    float ch[8]; double dh[8]; unsigned ih[8];
    for (int i = 0; i < 8; ++i) { ch[i] = threadIdx.x + i; dh[i] = ch[i]; ih[i] = threadIdx.x + i; }
    for (int it = 0; it < iters; ++it) {
        constexpr int STEPS = 8;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
#pragma unroll
            for (int i = s * NV / STEPS; i < (s + 1) * NV / STEPS; ++i) {
                const int c = i % 8;
                if (VK == 0) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(ch[c]) : "v"(b), "v"(a));
                if (VK == 1) asm volatile("v_add_u32 %0, %0, %1" : "+v"(ih[c]) : "v"(ih[(c + 1) % 8]));
                if (VK == 2) asm volatile("v_cndmask_b32 %0, %0, %1, vcc" : "+v"(ih[c]) : "v"(ih[(c + 1) % 8]) : );
                if (VK == 3) asm volatile("v_fma_f64 %0, %0, %1, %2" : "+v"(dh[c]) : "v"(bd), "v"(ad));
                if (VK == 4) asm volatile("v_cvt_f64_f32 %0, %1" : "=v"(dh[c]) : "v"(ch[c]));
                if (VK == 5) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(ch[c]) : "v"(b));
                if (VK == 6) asm volatile("v_lshl_add_u32 %0, %0, 1, %1" : "+v"(ih[c]) : "v"(ih[(c + 1) % 8]));
                if (VK == 7) asm volatile("v_cmp_lt_f32 vcc, %0, %1" :: "v"(ch[c]), "v"(b) : "vcc");
                if (VK == 8) asm volatile("v_add_f32 %0, %0, %1" : "+v"(ch[c]) : "v"(b));
                if (VK == 9) asm volatile("v_cvt_i32_f32 %0, %1" : "=v"(ih[c]) : "v"(ch[c]));
                if (VK == 10) asm volatile("v_mad_u32_u24 %0, %0, %1, %2" : "+v"(ih[c]) : "v"(ih[(c + 1) % 8]), "v"(ih[(c + 2) % 8]));
                if (VK == 11) asm volatile("v_med3_f32 %0, %0, %1, %2" : "+v"(ch[c]) : "v"(b), "v"(a));
                if (VK == 12) asm volatile("v_floor_f32 %0, %1" : "=v"(ch[c]) : "v"(ch[(c + 1) % 8]));
            }
#pragma unroll
            for (int i = s * NM / STEPS; i < (s + 1) * NM / STEPS; ++i) {
                if (MK == 1) {
                    if (i & 1) asm volatile("v_mfma_f32_32x32x2_f32 %0, %1, %2, %0" : "+v"(acc1) : "v"(a), "v"(b));
                    else       asm volatile("v_mfma_f32_32x32x2_f32 %0, %1, %2, %0" : "+v"(acc0) : "v"(a), "v"(b));
                }
                if (MK == 2) {
                    if (i & 1) asm volatile("v_mfma_f32_16x16x4_f32 %0, %1, %2, %0" : "+v"(b1) : "v"(a), "v"(b));
                    else       asm volatile("v_mfma_f32_16x16x4_f32 %0, %1, %2, %0" : "+v"(b0) : "v"(a), "v"(b));
                }
                if (MK == 3) {
                    if (i & 1) asm volatile("v_mfma_f64_16x16x4_f64 %0, %1, %2, %0" : "+v"(c1) : "v"(ad), "v"(bd));
                    else       asm volatile("v_mfma_f64_16x16x4_f64 %0, %1, %2, %0" : "+v"(c0) : "v"(ad), "v"(bd));
                }
                if (MK == 4) {          // four bfloat16 per lane and operand: a 64-bit register pair each
                    if (i & 1) asm volatile("v_mfma_f32_32x32x8_bf16 %0, %1, %2, %0" : "+v"(acc1) : "v"(ad), "v"(bd));
                    else       asm volatile("v_mfma_f32_32x32x8_bf16 %0, %1, %2, %0" : "+v"(acc0) : "v"(ad), "v"(bd));
                }
                if (MK == 5) {          // eight bfloat16 per lane and operand: four registers each
                    if (i & 1) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc1) : "v"(b0), "v"(b1));
                    else       asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc0) : "v"(b0), "v"(b1));
                }
                if (MK == 6) {
                    if (i & 1) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc1) : "v"(b0), "v"(b1));
                    else       asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc0) : "v"(b0), "v"(b1));
                }
                if (MK == 7) {
                    if (i & 1) asm volatile("v_mfma_f32_32x32x2_f32 %0, %1, %2, %0" : "+a"(acc1) : "v"(a), "v"(b));
                    else       asm volatile("v_mfma_f32_32x32x2_f32 %0, %1, %2, %0" : "+a"(acc0) : "v"(a), "v"(b));
                }
            }
        }
    }
    float r = 0;
    for (int i = 0; i < 16; ++i) r += acc0[i] + acc1[i];
    for (int i = 0; i < 4; ++i) r += b0[i] + b1[i] + (float)c0[i] + (float)c1[i];
    for (int i = 0; i < 8; ++i) r += ch[i] + (float)dh[i] + (float)ih[i];
    if (r == 123.456f) out[0] = r;
}
static float* d_out;
template <int MK, int NM, int VK, int NV, int NT>
float run() {
    auto kern = k<MK, NM, VK, NV, NT>;
    const int iters = 4000;
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    hipLaunchKernelGGL(kern, dim3(256), dim3(NT), 0, 0, 10, d_out);
    CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0));
    hipLaunchKernelGGL(kern, dim3(256), dim3(NT), 0, 0, iters, d_out);
    CK(hipEventRecord(e1)); CK(hipDeviceSynchronize());
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    return ms * 1e6f / iters;      // ns per iteration
}
static const char* vname[] = {"v_fma_f32", "v_add_u32", "v_cndmask_b32", "v_fma_f64", "v_cvt_f64_f32", "v_mul_f32", "v_lshl_add_u32", "v_cmp_lt_f32", "v_add_f32", "v_cvt_i32_f32", "v_mad_u32_u24", "v_med3_f32", "v_floor_f32"};
template <int MK, int NM, int VK, int NT>
void row(const char* mname) {
    const float m = run<MK, NM, VK, 0, NT>(), v = run<0, 0, VK, 64, NT>(), both = run<MK, NM, VK, 64, NT>();
    printf("%-16s x%d + %-15s x64  waves/SIMD=%d : mfma %7.1f ns  valu %7.1f ns (%.2f ns each)  both %7.1f ns  (sum %7.1f, overlap %4.0f %% of the shorter)\n", mname, NM, vname[VK], NT / 256, m, v, v / 64 / (NT / 256),
           both, m + v, 100.f * (m + v - both) / (m < v ? m : v));
    fflush(stdout);
}
template <int VK> void rows() {
    row<1, 8, VK, 512>("mfma 32x32x2 f32");
    row<1, 8, VK, 1024>("mfma 32x32x2 f32");
}
int main() {
    CK(hipMalloc(&d_out, 64));
    rows<0>(); rows<1>(); rows<3>(); rows<4>(); rows<5>(); rows<6>(); rows<7>(); rows<8>(); rows<9>(); rows<10>(); rows<11>(); rows<12>();
    row<2, 16, 0, 512>("mfma 16x16x4 f32"); row<2, 16, 0, 1024>("mfma 16x16x4 f32"); row<2, 16, 1, 1024>("mfma 16x16x4 f32");
    // 16-bit matrix instructions (f32 accumulation) beside vector work: do they share the issue port too?
    row<4, 8, 0, 512>("mfma 32x32x8 bf16"); row<4, 8, 0, 1024>("mfma 32x32x8 bf16"); row<4, 8, 1, 1024>("mfma 32x32x8 bf16"); row<4, 8, 9, 1024>("mfma 32x32x8 bf16");
    row<5, 8, 0, 512>("mfma 32x32x16bf16"); row<5, 8, 0, 1024>("mfma 32x32x16bf16"); row<5, 8, 1, 1024>("mfma 32x32x16bf16"); row<5, 8, 9, 1024>("mfma 32x32x16bf16");
    row<6, 8, 0, 512>("32x32x16bf16 agpr"); row<6, 8, 0, 1024>("32x32x16bf16 agpr"); row<6, 8, 1, 1024>("32x32x16bf16 agpr");
    row<7, 8, 0, 512>("32x32x2 f32 agpr"); row<7, 8, 0, 1024>("32x32x2 f32 agpr");
    row<3, 16, 0, 512>("mfma 16x16x4 f64"); row<3, 16, 0, 1024>("mfma 16x16x4 f64"); row<3, 16, 1, 1024>("mfma 16x16x4 f64"); row<3, 16, 3, 1024>("mfma 16x16x4 f64");
    return 0;
}
