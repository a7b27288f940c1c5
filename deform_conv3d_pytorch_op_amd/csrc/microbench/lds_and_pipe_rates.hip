// LDS instruction rates and pipe overlap on gfx950: the measurements the kernels' cost model rests on.
// Instruction mixes are pinned with inline asm; 256 workgroups (one per CU), 4000 iterations each.
// Build and run (no arguments):
//   hipcc --offload-arch=gfx950 -O3 -Xclang -target-feature -Xclang -packed-fp32-ops -o lds_and_pipe_rates lds_and_pipe_rates.hip
// Every LDS address comes from a host table with values below 64 KB; the workgroup allocates 128 KB
// (or 64 KB with two workgroups per CU), so no access can leave the allocation.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <vector>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1); } } while (0)
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef float f2v __attribute__((ext_vector_type(2)));

// per iteration: NM mfma (round robin over 2 accumulators), NV v_fma_f32 (8 chains), NL lds ops of kind LK
// LK: 0 none, 1 ds_read_b32, 2 ds_read_b64, 3 ds_read_b128, 4 ds_add_u32, 5 ds_add_u64, 6 ds_add_f32, 7 ds_add_f64, 8 ds_write_b32, 9 ds_write_b64
// ORDER: 0 = lds, valu, mfma blocks ; 1 = interleaved finely
template <int NM, int NV, int NL, int LK, int NT>
__global__ __launch_bounds__(NT) void k(const unsigned* __restrict__ idx, int iters, float* out, long long* clk) {
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned* c32 = reinterpret_cast<unsigned*>(smem);
    for (int i = threadIdx.x; i < 32768; i += NT) c32[i] = 0;
    __syncthreads();
    unsigned la[8];
    for (int i = 0; i < 8; ++i) la[i] = idx[threadIdx.x * 8 + i];     // byte addresses
    f16v acc0 = {0}, acc1 = {0};
    float a = threadIdx.x * 1e-3f, b = 1.0001f;
    float ch[8];
    for (int i = 0; i < 8; ++i) ch[i] = threadIdx.x + i;
    f4v r4[4]; f2v r2[4]; float r1[8];
    for (int i = 0; i < 4; ++i) { r4[i] = f4v{0,0,0,0}; r2[i] = f2v{0,0}; }
    for (int i = 0; i < 8; ++i) r1[i] = 0;
    unsigned long long v64 = threadIdx.x + 1; unsigned v32 = threadIdx.x + 1; float vf = 1.f; double vd = 1.0;
    const long long t0 = clock64();
    for (int it = 0; it < iters; ++it) {
        constexpr int STEPS = 8;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            // LDS ops of this step
#pragma unroll
            for (int i = s * NL / STEPS; i < (s + 1) * NL / STEPS; ++i) {
                const unsigned ad = la[i % 8];
                if (LK == 1) asm volatile("ds_read_b32 %0, %1" : "=v"(r1[i % 8]) : "v"(ad));
                if (LK == 2) asm volatile("ds_read_b64 %0, %1" : "=v"(r2[i % 4]) : "v"(ad));
                if (LK == 3) asm volatile("ds_read_b128 %0, %1" : "=v"(r4[i % 4]) : "v"(ad));
                if (LK == 4) asm volatile("ds_add_u32 %0, %1" :: "v"(ad), "v"(v32));
                if (LK == 5) asm volatile("ds_add_u64 %0, %1" :: "v"(ad), "v"(v64));
                if (LK == 6) asm volatile("ds_add_f32 %0, %1" :: "v"(ad), "v"(vf));
                if (LK == 7) asm volatile("ds_add_f64 %0, %1" :: "v"(ad), "v"(vd));
                if (LK == 8) asm volatile("ds_write_b32 %0, %1" :: "v"(ad), "v"(v32));
                if (LK == 9) asm volatile("ds_write_b64 %0, %1" :: "v"(ad), "v"(v64));
            }
#pragma unroll
            for (int i = s * NV / STEPS; i < (s + 1) * NV / STEPS; ++i)
                asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(ch[i % 8]) : "v"(b), "v"(a));
#pragma unroll
            for (int i = s * NM / STEPS; i < (s + 1) * NM / STEPS; ++i) {
                if (i & 1) asm volatile("v_mfma_f32_32x32x2_f32 %0, %1, %2, %0" : "+v"(acc1) : "v"(a), "v"(b));
                else       asm volatile("v_mfma_f32_32x32x2_f32 %0, %1, %2, %0" : "+v"(acc0) : "v"(a), "v"(b));
            }
        }
        if (LK >= 1 && LK <= 3) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const long long t1 = clock64();
    float r = 0;
    for (int i = 0; i < 16; ++i) r += acc0[i] + acc1[i];
    for (int i = 0; i < 8; ++i) r += ch[i] + r1[i];
    for (int i = 0; i < 4; ++i) r += r4[i][0] + r4[i][3] + r2[i][0] + r2[i][1];
    if (r == 123.456f) out[0] = r;
    if (blockIdx.x == 0 && threadIdx.x == 0) clk[0] = t1 - t0;
}

static unsigned* d_idx_lin; static unsigned* d_idx_rnd; static float* d_out; static long long* d_clk;

template <int NM, int NV, int NL, int LK, int NT>
void run(const char* name, bool rnd, int wgs_per_cu = 1) {
    const size_t lds = 131072 / wgs_per_cu;
    auto kern = k<NM, NV, NL, LK, NT>;
    CK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    const int iters = 4000;
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    const unsigned* ix = rnd ? d_idx_rnd : d_idx_lin;
    hipLaunchKernelGGL(kern, dim3(256 * wgs_per_cu), dim3(NT), lds, 0, ix, 10, d_out, d_clk);
    CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0));
    hipLaunchKernelGGL(kern, dim3(256 * wgs_per_cu), dim3(NT), lds, 0, ix, iters, d_out, d_clk);
    CK(hipEventRecord(e1)); CK(hipDeviceSynchronize());
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    long long c; CK(hipMemcpy(&c, d_clk, 8, hipMemcpyDeviceToHost));
    const int wps = NT / 256 * wgs_per_cu;      // waves per SIMD
    printf("%-34s %s w/SIMD=%d  M=%2d V=%3d L=%2d | %7.3f ms  %8.1f clk64/iter  %8.1f cyc@2.4GHz/iter\n", name, rnd ? "rnd" : "lin", wps, NM, NV, NL,
           ms, (double)c / iters, ms * 1e-3 * 2.4e9 / iters);
    fflush(stdout);
}

int main() {
    std::vector<unsigned> lin(1024 * 8), rnd(1024 * 8);
    srand(1);
    for (int t = 0; t < 1024; ++t)
        for (int i = 0; i < 8; ++i) {
            lin[t * 8 + i] = ((t % 64) * 16 + i * 1024 + (t / 64) * 8192) % 65536;      // 16-byte slots, conflict free for every width
            rnd[t * 8 + i] = (rand() % 4096) * 16;
        }
    CK(hipMalloc(&d_idx_lin, lin.size() * 4)); CK(hipMalloc(&d_idx_rnd, rnd.size() * 4));
    CK(hipMalloc(&d_out, 64)); CK(hipMalloc(&d_clk, 64));
    CK(hipMemcpy(d_idx_lin, lin.data(), lin.size() * 4, hipMemcpyHostToDevice));
    CK(hipMemcpy(d_idx_rnd, rnd.data(), rnd.size() * 4, hipMemcpyHostToDevice));
    printf("== pipes alone, 1 / 2 / 4 waves per SIMD ==\n");
    run<8, 0, 0, 0, 256>("mfma x8", false);
    run<8, 0, 0, 0, 512>("mfma x8", false);
    run<8, 0, 0, 0, 1024>("mfma x8", false);
    run<0, 64, 0, 0, 256>("valu x64", false);
    run<0, 64, 0, 0, 512>("valu x64", false);
    run<0, 64, 0, 0, 1024>("valu x64", false);
    printf("== mfma + valu in the same wave ==\n");
    run<8, 64, 0, 0, 256>("mfma x8 + valu x64", false);
    run<8, 64, 0, 0, 512>("mfma x8 + valu x64", false);
    run<8, 64, 0, 0, 1024>("mfma x8 + valu x64", false);
    run<8, 128, 0, 0, 256>("mfma x8 + valu x128", false);
    run<8, 128, 0, 0, 512>("mfma x8 + valu x128", false);
    run<8, 128, 0, 0, 1024>("mfma x8 + valu x128", false);
    run<8, 32, 0, 0, 1024>("mfma x8 + valu x32", false);
    printf("== LDS alone (16 waves/CU unless noted) ==\n");
    run<0, 0, 32, 1, 1024>("ds_read_b32", false);  run<0, 0, 32, 1, 1024>("ds_read_b32", true);
    run<0, 0, 32, 2, 1024>("ds_read_b64", false);  run<0, 0, 32, 2, 1024>("ds_read_b64", true);
    run<0, 0, 32, 3, 1024>("ds_read_b128", false); run<0, 0, 32, 3, 1024>("ds_read_b128", true);
    run<0, 0, 32, 4, 1024>("ds_add_u32", false);   run<0, 0, 32, 4, 1024>("ds_add_u32", true);
    run<0, 0, 32, 5, 1024>("ds_add_u64", false);   run<0, 0, 32, 5, 1024>("ds_add_u64", true);
    run<0, 0, 32, 6, 1024>("ds_add_f32", false);   run<0, 0, 32, 6, 1024>("ds_add_f32", true);
    run<0, 0, 32, 7, 1024>("ds_add_f64", false);   run<0, 0, 32, 7, 1024>("ds_add_f64", true);
    run<0, 0, 32, 8, 1024>("ds_write_b32", false); run<0, 0, 32, 8, 1024>("ds_write_b32", true);
    run<0, 0, 32, 9, 1024>("ds_write_b64", false); run<0, 0, 32, 9, 1024>("ds_write_b64", true);
    run<0, 0, 32, 5, 512>("ds_add_u64 8 waves", true);
    run<0, 0, 32, 5, 256>("ds_add_u64 4 waves", true);
    run<0, 0, 32, 4, 512>("ds_add_u32 8 waves", true);
    printf("== LDS + other pipes ==\n");
    run<0, 64, 32, 5, 1024>("ds_add_u64 x32 + valu x64", true);
    run<8, 0, 32, 5, 1024>("ds_add_u64 x32 + mfma x8", true);
    run<8, 64, 32, 5, 1024>("ds_add_u64 x32 + mfma x8 + valu x64", true);
    run<8, 64, 32, 5, 512>("ds_add_u64 x32 + mfma x8 + valu x64", true);
    run<8, 64, 32, 4, 1024>("ds_add_u32 x32 + mfma x8 + valu x64", true);
    run<8, 64, 8, 3, 1024>("ds_read_b128 x8 + mfma x8 + valu x64", true);
    run<8, 32, 8, 3, 1024>("ds_read_b128 x8 + mfma x8 + valu x32", true);
    run<8, 32, 8, 3, 512>("ds_read_b128 x8 + mfma x8 + valu x32", true);
    return 0;
}
