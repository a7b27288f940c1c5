// C ABI of libdcn_amd.so (declared in include/dcn_amd.h): argument validation, workspace
// layout and kernel launches.  No device memory is allocated here and nothing synchronises; all
// work is enqueued on the caller's stream.
#include "../../include/dcn_amd.h"
#include "dcn_kernels.h"
#include "dcn_forward.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <type_traits>
#include <utility>

namespace {

using namespace dcn;

thread_local std::string g_err;

int fail(int code, const char* msg) {
    g_err = msg;
    return code;
}


// Largest re-laid-out weight any call needs; see relayout_weight_kernel for the two layouts.
template <typename T> void fwd_weight_pad(int M, int Cg, int& MT, int& mchunks, int& Mp, int& Cgp) {
    const int TN = Mma<T>::TN, KL = Mma<T>::KL;
    const int mtiles = (M + TN - 1) / TN;
    MT = mtiles >= 8 ? 8 : (mtiles > 2 ? 4 : mtiles);          // 1, 2, 4 or 8 tiles per wavefront
    mchunks = (mtiles + MT - 1) / MT;
    Mp = mchunks * MT * TN;
    Cgp = Cg + 2 * KL;       // the kernels read up to one reduction step past the last channel
}
// backward-data layout.  MK = reduction steps over output channels whose grad_output values
// backward_data_kernel keeps in registers (0: M too large, the kernel re-reads grad_output per tap).
template <typename T> int bwd_data_mk(int M) {
    const int steps = (M + Mma<T>::KL - 1) / Mma<T>::KL;
    for (int mk = 8; mk <= 64; mk *= 2)
        if (steps <= mk) return mk;
    return 0;
}
template <typename T> void bwd_data_weight_pad(int M, int Cg, int& Mp, int& Cgp) {
    // rows: reduction steps are consumed in batches of 8; the coordinate kernel reads up to KL rows further
    const int KL = Mma<T>::KL;
    const int steps = ((M + KL - 1) / KL + 7) / 8 * 8;
    Mp = steps * KL + KL;
    const int mk = bwd_data_mk<T>(M) * KL;
    if (mk > Mp) Mp = mk;
    Cgp = Cg + Mma<T>::TN;
}
size_t align256(size_t v) { return (v + 255) / 256 * 256; }

constexpr int TAP_PAD = 8;      // zero tap slabs behind the last group: an MFMA pass may start up to 7 taps before the end
// Elements of the per-chunk weight slabs of the fused backward kernel (pack_weight_kernel, chunks of
// `cch` channels) for `slabs` slabs.
template <typename T, typename S = T> size_t packed_weight_elems(int M, int kV, size_t slabs, int cch) {
    const int TP = Mma<T>::TN / cch;
    return slabs * ((kV + TP - 1) / TP) * (size_t)gcol_slab_steps<T, S>(M) * 64 * (std::is_same<S, T>::value ? 1 : 4);
}
// Upper bound of chunk_slot<cch>(cpg, Cg, c) + 1 over the channels: the slabs a per-chunk weight
// layout occupies.  cpg = 0: the channels per deformable group are not known (the first workspace
// query is not told them) and the bound assumes their largest possible number of groups, C_in.
size_t slab_bound(size_t C_in, int G, int cpg, int cch) { return C_in / cch + (cpg > 0 ? C_in / cpg : C_in) + G + 1; }
// Either weight layout of backward_input_offset fits.
template <typename T> size_t bwd_data_weight_bytes(int M, int Cg, int kV, int G, int cpg = 0) {
    int Mp, Cgp;
    bwd_data_weight_pad<T>(M, Cg, Mp, Cgp);
    const size_t plain = ((size_t)G * kV + TAP_PAD) * Mp * Cgp;
    const size_t C_in = (size_t)Cg * G;
    const size_t packed4 = packed_weight_elems<T>(M, kV, slab_bound(C_in, G, cpg, 4), 4);
    const size_t packed8 = packed_weight_elems<T>(M, kV, slab_bound(C_in, G, cpg, 8), 8);
    const size_t packed16 = packed_weight_elems<T>(M, kV, slab_bound(C_in, G, cpg, 16), 16);
    size_t packed = packed4 > packed8 ? packed4 : packed8;
    if (packed16 > packed) packed = packed16;
    return align256((plain > packed ? plain : packed) * sizeof(T));
}
// Partial outputs of a forward pass that splits the input channels of a position block over several
// workgroups: only layers of few positions do (too few blocks to fill the device), with at most
// FWD_MAX_SPLIT parts and FWD_PARTIAL_CAP bytes.
constexpr int FWD_MAX_SPLIT = 16;
constexpr size_t FWD_PARTIAL_CAP = (size_t)64 << 20;
constexpr size_t FWD_SPLIT_POSITIONS = 256 * 512;      // no split from this many positions on: they fill the device anyway
size_t forward_partial_bound(int N, int C_out, size_t outV, size_t elem) {
    if ((size_t)N * outV >= FWD_SPLIT_POSITIONS) return 0;
    const size_t all = (size_t)FWD_MAX_SPLIT * N * C_out * outV * elem;
    return align256(all < FWD_PARTIAL_CAP ? all : FWD_PARTIAL_CAP) + 256;
}
template <typename T> size_t workspace_need(int N, int C_in, int C_out, size_t inV, size_t outV, int kV, int G, int cpg = 0) {
    const int M = C_out / G, Cg = C_in / G;
    int MT, mchunks, Mp, Cgp;
    fwd_weight_pad<T>(M, Cg, MT, mchunks, Mp, Cgp);
    // forward: [g][tap][c][m] for the kernel without LDS tiling, or one slab per four channels for the
    // halo kernel (its row padding is at most eight tiles' worth)
    const int TNf = Mma<T>::TN;
    const int Mp8 = ((M + TNf - 1) / TNf + 7) / 8 * 8 * TNf;
    const size_t fwd_plain = (size_t)G * kV * (Mp > Mp8 ? Mp : Mp8) * Cgp * sizeof(T);
    const size_t fwd_quad = slab_bound((size_t)C_in, G, cpg, FQ) * forward_slab_elems<T>(kV, Mp8) * sizeof(T);
    const size_t fwd = (fwd_plain > fwd_quad ? fwd_plain : fwd_quad) + forward_partial_bound(N, C_out, outV, sizeof(T));
    // (+ the last whole 256-byte block of the workspace: weight bounds and the plan the device chose)
    const size_t bwd = bwd_data_weight_bytes<T>(M, Cg, kV, G, cpg) + 2 * align256((size_t)N * C_in * inV * sizeof(T)) + 512;
    // backward_weight: two channels-last copies + one partial weight per position split (at most 256 splits,
    // and never more than about 4096 workgroups: see bww_plan)
    const int TNq = Mma<T>::TN;
    const long long tiles_lb = (long long)kV * ((C_in + TNq - 1) / TNq);           // lower bound of kV * nct * mchunks
    long long split_ub = (4096 + tiles_lb - 1) / tiles_lb;
    if (split_ub > 256) split_ub = 256;
    if (split_ub < 1) split_ub = 1;
    const size_t bww = align256((size_t)N * C_in * inV * sizeof(T)) + align256((size_t)N * C_out * outV * sizeof(T)) +
                       align256((size_t)split_ub * kV * C_out * Cg * sizeof(T));
    size_t need = fwd > bwd ? fwd : bwd;
    return need > bww ? need : bww;
}

struct Geometry {   // the reference's argument list, 2-D mapped onto slots 1,2 with a unit length axis
    int nd, N, C_in, C_out, in[3], out[3], k[3], pad[3], stride[3], dil[3], cpg, G;
};

// Mirrors shape_check of the reference as far as it can be stated without tensor handles
// (deform3d/lib/deform_conv3d_cuda.cpp:24-87): the extents must be consistent with each other and
// with the output-size formula.  Rank and per-tensor size checks live in the Python front end,
// which owns the tensors.
int validate(const Geometry& g, Params& P) {
    if (g.N <= 0 || g.C_in <= 0 || g.C_out <= 0) return fail(DCN_E_ARGUMENT, "batch / channel extents must be positive");
    if (g.G <= 0 || g.C_in % g.G || g.C_out % g.G) return fail(DCN_E_ARGUMENT, "input c != kernel c");
    if (g.cpg <= 0 || g.C_in % g.cpg) return fail(DCN_E_ARGUMENT, "off channel");
    static const char* const omsg[3] = {"error output ll", "error outhh", "error outww"};
    for (int a = 3 - g.nd; a < 3; ++a) {
        if (g.in[a] <= 0 || g.k[a] <= 0 || g.stride[a] <= 0 || g.dil[a] <= 0 || g.pad[a] < 0)
            return fail(DCN_E_ARGUMENT, "input / kernel / stride / dilation extents must be positive, pad non-negative");
        if (g.in[a] + 2 * g.pad[a] - g.k[a] < 0) return fail(DCN_E_ARGUMENT, omsg[a]);
        // the reference's dilation-blind output size, or the usual dilation-aware one (the sampler
        // gives every position a meaning, so both are served)
        const int blind = (g.in[a] + 2 * g.pad[a] - g.k[a]) / g.stride[a] + 1;
        const int span = g.in[a] + 2 * g.pad[a] - g.dil[a] * (g.k[a] - 1) - 1;
        const int standard = span >= 0 ? span / g.stride[a] + 1 : 0;
        if (g.out[a] != blind && !(standard >= 1 && g.out[a] == standard)) return fail(DCN_E_ARGUMENT, omsg[a]);
    }
    const long long inV = (long long)g.in[0] * g.in[1] * g.in[2], outV = (long long)g.out[0] * g.out[1] * g.out[2];
    // per-channel offsets are 32-bit inside the kernels (including a bias of up to 4 channels)
    if (inV > (1ll << 27) || outV > (1ll << 27)) return fail(DCN_E_ARGUMENT, "a single channel exceeds 2^27 voxels");
    // channels-last voxel*channel offsets of one sample are 32-bit as well
    if (inV * g.C_in > (1ll << 31)) return fail(DCN_E_ARGUMENT, "one input sample exceeds 2^31 elements");
    if (g.N > 65535) return fail(DCN_E_ARGUMENT, "batch exceeds 65535");
    P.oob_zero = 0;
    P.nd = g.nd; P.N = g.N; P.C_in = g.C_in; P.C_out = g.C_out; P.G = g.G; P.cpg = g.cpg; P.DG = g.C_in / g.cpg;
    P.M = g.C_out / g.G; P.Cg = g.C_in / g.G;
    for (int a = 0; a < 3; ++a) {
        P.in[a] = g.in[a]; P.out[a] = g.out[a]; P.k[a] = g.k[a];
        P.pad[a] = g.pad[a]; P.stride[a] = g.stride[a]; P.dil[a] = g.dil[a];
    }
    P.inV = (unsigned)inV; P.outV = (unsigned)outV; P.kV = g.k[0] * g.k[1] * g.k[2];
    P.tiles = P.mchunks = P.Mp = P.Cgp = P.nsplit = P.nctiles = 0;
    return DCN_OK;
}

int check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        g_err = std::string(what) + ": " + hipGetErrorString(e);
        return DCN_E_LAUNCH;
    }
    return DCN_OK;
}

template <typename T>
int relayout(const Params& P, const T* w, T* wt, int channel_fastest, hipStream_t s) {
    const size_t total = (size_t)P.G * P.kV * P.Mp * P.Cgp;
    const int blocks = (int)((total + 255) / 256 > 4096 ? 4096 : (total + 255) / 256);
    hipLaunchKernelGGL(relayout_weight_kernel<T>, dim3(blocks), dim3(256), 0, s, P, w, wt, channel_fastest);
    return check_launch("relayout_weight_kernel");
}

// ---------------------------------------------------------------------------------------------
// Halo tiling plan: block of output positions per workgroup, halo extents, channels per LDS pass.
// Returns false when the geometry does not suit (halo too large for the staging table or LDS).
// Tuning knobs (environment, read once per process):
//   DCN_HALO_MARGIN        voxels of halo beyond the integer tap span on each side: one fixed margin instead of
//                          the choice on the device among 2, 3, 4 (3-D) or 2, 4, 6 (2-D)
//   DCN_ADAPTIVE_MARGIN=0  always the smallest of those margins (2)
//   DCN_TRACE_PLANS=1      print the halo plans and launches of every call on stderr
//   DCN_LDS_BUDGET_KB      LDS per 512-thread workgroup of the forward halo kernel (default 72: two per CU)
//   DCN_FORWARD_WG=512     never use the 1024-thread forward variant; =1024 use it whenever its halo fits
//   DCN_FORWARD_SPLIT=n    forward pass: split the input channels of a position block over at most n workgroups (0: never)
//   DCN_FORWARD_TAIL=0     forward pass: never split only the units of the last, partly filled round of workgroups (n > 1: n ways)
//   DCN_FORWARD_TAIL2=0    forward pass: the split units of the last round all the same number of ways, never in two runs
//   DCN_FORWARD_SLOTS=n    forward pass: plan the launch as if n workgroups ran at once (test hook)
//   DCN_SCATTER_BUDGET_KB  LDS per workgroup of the privatised scatter kernel (default 144)
//   DCN_SCATTER=global     scatter grad-input with global atomics instead of the LDS-privatised kernel
//   DCN_COORD=separate     grad_offset from the channels-last kernel instead of the fused LDS-halo kernel
//   DCN_FUSED_WAVES=4      fused backward kernel with four wavefronts per workgroup even where eight fit
//   DCN_FUSED_CHUNK=4      fused backward kernel with 4-channel chunks also where it would take 8 or 16; =8: never 16 (2-D layers)
//   DCN_FUSED_TAIL=0       fused backward kernel: all items split alike, never only those of the last round
//   DCN_CSPLIT=n           fused backward kernel: every item split over n workgroups
//   DCN_FUSED_SLOTS=n      fused backward kernel: plan the launch as if n workgroups ran at once (test hook)
//   DCN_FUSED_FIXED=0      fused backward kernel: runtime plane stride even where the compile-time one fits
//   DCN_FUSED_PAIR=0       fused backward kernel, float32: one channel per 64-bit LDS cell instead of two 32-bit halves
//   DCN_FUSED_BREG2=0      fused backward kernel: no second register set for the grad_output operand of 64 < M <= 128
//   DCN_GLOBAL_PLAN=0      backward_input_offset (3-D): the device is not offered the path without LDS tiling
//   DCN_NATIVE16=0         16-bit entry points: always widen to float32 and run the float32 kernels
static size_t env_kb(const char* name, int dflt) {
    const char* e = getenv(name);
    const int v = e ? atoi(e) : dflt;
    return (size_t)(v > 0 ? v : dflt) * 1024;
}
static size_t lds_budget() { static const size_t v = env_kb("DCN_LDS_BUDGET_KB", 72); return v; }
static size_t scatter_budget() { static const size_t v = env_kb("DCN_SCATTER_BUDGET_KB", 144); return v; }
static bool fused_coord() {
    static const int v = [] { const char* e = getenv("DCN_COORD"); return (e && strcmp(e, "separate") == 0) ? 0 : 1; }();
    return v != 0;
}
// What the library needs to know about a GPU, looked up once per device ordinal.
struct DeviceInfo { int state = 0; int cus = 256; };      // state: 0 not looked up, 1 usable, -1 not a gfx950
constexpr int MAX_DEVICES = 64;
std::mutex g_device_lock;
DeviceInfo g_device[MAX_DEVICES];

// Fills `out` for the current device; DCN_E_DEVICE when there is none or it is not a gfx950.
int device_info(const DeviceInfo** out, int* ordinal = nullptr) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
        (void)hipGetLastError();
        return fail(DCN_E_DEVICE, "no current HIP device (or its ordinal is beyond 63)");
    }
    std::lock_guard<std::mutex> lock(g_device_lock);
    DeviceInfo& d = g_device[dev];
    if (d.state == 0) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
            (void)hipGetLastError();
            return fail(DCN_E_DEVICE, "hipGetDeviceProperties failed");
        }
        d.state = strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : -1;
        if (prop.multiProcessorCount > 0) d.cus = prop.multiProcessorCount;
    }
    if (d.state < 0) return fail(DCN_E_DEVICE, "the current device is not a gfx950 GPU");
    if (out) *out = &d;
    if (ordinal) *ordinal = dev;
    return DCN_OK;
}
static int cu_count() {      // of the current device (every entry point has called device_info by then)
    const DeviceInfo* d = nullptr;
    return device_info(&d) == DCN_OK ? d->cus : 256;
}
static int wide_forward() {      // 0 never, 1 when it pays, 2 whenever the halo fits
    static const int v = [] {
        const char* e = getenv("DCN_FORWARD_WG");
        return !e ? 1 : atoi(e) == 512 ? 0 : atoi(e) == 1024 ? 2 : 1;
    }();
    return v;
}
static bool fused_chunk16() {     // DCN_FUSED_CHUNK=8 (or 4): never take 16-channel chunks in the fused backward kernel
    static const int v = [] { const char* e = getenv("DCN_FUSED_CHUNK"); return (e && (atoi(e) == 8 || atoi(e) == 4)) ? 0 : 1; }();
    return v != 0;
}
static bool fused_chunk8() {      // DCN_FUSED_CHUNK=4: never take 8-channel chunks in the fused backward kernel
    static const int v = [] { const char* e = getenv("DCN_FUSED_CHUNK"); return (e && atoi(e) == 4) ? 0 : 1; }();
    return v != 0;
}
static int fused_first_waves() {
    static const int v = [] { const char* e = getenv("DCN_FUSED_WAVES"); return (e && atoi(e) == 4) ? 4 : 8; }();
    return v;
}
static bool fused_fixed_stride() {      // DCN_FUSED_FIXED=0: runtime plane stride even where the compile-time one fits
    static const int v = [] { const char* e = getenv("DCN_FUSED_FIXED"); return (e && atoi(e) == 0) ? 0 : 1; }();
    return v != 0;
}
static bool fused_tail_split() {        // DCN_FUSED_TAIL=0: the fused backward kernel never splits only the items of the last round
    static const int v = [] { const char* e = getenv("DCN_FUSED_TAIL"); return (e && atoi(e) == 0) ? 0 : 1; }();
    return v != 0;
}
static int forced_slots() {             // DCN_FUSED_SLOTS=n (test hook): plan the fused backward launch as if n workgroups ran at once
    static const int v = [] { const char* e = getenv("DCN_FUSED_SLOTS"); return e && atoi(e) > 0 ? atoi(e) : 0; }();
    return v;
}
static int forward_split() {            // DCN_FORWARD_SPLIT=n: the forward pass splits the input channels of a position block at most n ways
    static const int v = [] { const char* e = getenv("DCN_FORWARD_SPLIT"); return e ? atoi(e) : 1 << 20; }();
    return v;
}
static int forward_slots() {            // DCN_FORWARD_SLOTS=n (test hook): plan the forward launch as if n workgroups ran at once
    static const int v = [] { const char* e = getenv("DCN_FORWARD_SLOTS"); return e && atoi(e) > 0 ? atoi(e) : 0; }();
    return v;
}
static int forward_tail_split() {       // DCN_FORWARD_TAIL=0: the forward pass never splits the units of its last round of workgroups; n > 1: n ways
    static const int v = [] { const char* e = getenv("DCN_FORWARD_TAIL"); return e ? atoi(e) : 1; }();
    return v;
}
static bool forward_tail_two_runs() {    // DCN_FORWARD_TAIL2=0: the split units of the forward pass's last round are all split the same number of ways
    static const int v = [] { const char* e = getenv("DCN_FORWARD_TAIL2"); return (e && atoi(e) == 0) ? 0 : 1; }();
    return v != 0;
}
static bool fused_pair() {              // DCN_FUSED_PAIR=0: float32 LDS cells of the fused backward kernel hold one channel each (64-bit)
    static const int v = [] { const char* e = getenv("DCN_FUSED_PAIR"); return (e && atoi(e) == 0) ? 0 : 1; }();
    return v != 0;
}
static bool fused_breg2() {             // DCN_FUSED_BREG2=0: grad_output operand in registers only up to 32 reduction steps
    static const int v = [] { const char* e = getenv("DCN_FUSED_BREG2"); return (e && atoi(e) == 0) ? 0 : 1; }();
    return v != 0;
}
static bool native16() {                // DCN_NATIVE16=0: the 16-bit entry points always widen to float32 first
    static const int v = [] { const char* e = getenv("DCN_NATIVE16"); return (e && atoi(e) == 0) ? 0 : 1; }();
    return v != 0;
}
static bool global_plan() {             // DCN_GLOBAL_PLAN=0: the device never chooses the path without LDS tiling
    static const int v = [] { const char* e = getenv("DCN_GLOBAL_PLAN"); return (e && atoi(e) == 0) ? 0 : 1; }();
    return v != 0;
}
static bool scatter_in_lds() {
    static const int v = [] { const char* e = getenv("DCN_SCATTER"); return (e && strcmp(e, "global") == 0) ? 0 : 1; }();
    return v != 0;
}
#define LDS_BUDGET lds_budget()
static int halo_margin() {      // DCN_HALO_MARGIN: one fixed margin; -1 when not set
    static const int v = [] {
        const char* e = getenv("DCN_HALO_MARGIN");
        if (!e) return -1;
        const int m = atoi(e);
        return m < 0 ? 0 : m;
    }();
    return v;
}
// Halo margins to plan for, ascending; the first is the one taken when nothing can be chosen.
static int plan_margins(int nd, int* m) {
    static const int adaptive = [] { const char* e = getenv("DCN_ADAPTIVE_MARGIN"); return (e && atoi(e) == 0) ? 0 : 1; }();
    if (halo_margin() >= 0) { m[0] = halo_margin(); return 1; }
    m[0] = 2;
    if (!adaptive) return 1;
    m[1] = nd == 3 ? 3 : 4;
    m[2] = nd == 3 ? 4 : 6;
    return MAX_PLANS;
}
static_assert(MAX_PLANS == 3, "plan_margins fills three margins");
static bool trace_plans() {             // DCN_TRACE_PLANS=1: the halo plans and launches of every call on stderr
    static const int v = [] { const char* e = getenv("DCN_TRACE_PLANS"); return (e && atoi(e) != 0) ? 1 : 0; }();
    return v != 0;
}
static int default_margin() { return halo_margin() >= 0 ? halo_margin() : 2; }
static int forced_csplit() {    // DCN_CSPLIT=n: workgroups per (tile, deformable group) of the fused backward kernel
    static const int v = [] { const char* e = getenv("DCN_CSPLIT"); return e && atoi(e) > 0 ? atoi(e) : 0; }();
    return v;
}

template <typename T, int ND>
bool plan_halo(Params& P, size_t budget, int m, int max_chunk = 1 << 30, size_t cell_bytes = sizeof(T), int waves = WAVESH,
               bool smallest_halo = false, int chunk_mult = 0, const int* blocks = nullptr, int wmult = 1) {
    const int npos = waves * Mma<T>::TN;        // positions per workgroup, one column tile per wavefront
    int td[3] = {1, 1, 1};
    if (ND == 3) { td[1] = 8; td[2] = 8; td[0] = npos / 64; }
    else         { td[2] = 16; td[1] = npos / 16; }
    if (blocks) {                               // the block shape of another plan
        for (int a = 0; a < 3; ++a) td[a] = blocks[a];
    } else if (smallest_halo) {
        // the block shape (powers of two, at least 4 positions along the fastest axis) with the
        // smallest halo: strided geometries want blocks that are short along the strided axes
        long long best = -1;
        for (int a = 1; a <= npos; a *= 2)
            for (int b = 1; a * b <= npos; b *= 2) {
                const int c = npos / (a * b);
                if (c < 4 || (ND == 2 && a != 1)) continue;
                const int cand[3] = {a, b, c};
                long long hv = 1;
                for (int x = 3 - ND; x < 3; ++x) hv *= (cand[x] - 1) * P.stride[x] + (P.k[x] - 1) * P.dil[x] + 1 + 2 * m;
                if (best < 0 || hv < best) { best = hv; td[0] = a; td[1] = b; td[2] = c; }
            }
    }
    long long hvol = 1, tiles = 1;
    for (int a = 0; a < 3; ++a) {
        P.tdim[a] = td[a];
        P.ntile[a] = (P.out[a] + td[a] - 1) / td[a];
        const bool used = a >= 3 - ND;
        P.mlo[a] = used ? m : 0;
        // lowest corner: base - m; highest corner: base + m (the high corner of a sample at base + m - eps)
        P.hext[a] = used ? (td[a] - 1) * P.stride[a] + (P.k[a] - 1) * P.dil[a] + 1 + 2 * m : 1;
        // (wmult: the innermost extent rounded up to a multiple, for kernels whose LDS layout depends on
        // the position of a halo voxel modulo that number; the extra cells lie on the high side)
        if (a == 2 && wmult > 1) P.hext[a] = (P.hext[a] + wmult - 1) / wmult * wmult;
        hvol *= P.hext[a];
        tiles *= P.ntile[a];
    }
    if (hvol > MAX_HVOL) return false;
    P.hvol = (int)hvol;
    P.hstride = ((int)hvol + 63) / 64 * 64 + 32;
    const int KL = chunk_mult > 0 ? chunk_mult : Mma<T>::KL;      // channels per pass come in multiples of this
    if (budget <= (size_t)hvol * 4) return false;
    long long cc = (long long)((budget - (size_t)hvol * 4) / ((size_t)P.hstride * cell_bytes));
    cc = cc / KL * KL;
    const int seg = P.cpg < P.Cg ? P.cpg : P.Cg;          // longest run of channels sharing offsets and group
    const int seg_up = (seg + KL - 1) / KL * KL;
    if (cc > seg_up) cc = seg_up;
    if (cc > max_chunk) cc = max_chunk / KL * KL;
    if (cc < KL) return false;
    P.cchunk = (int)cc;
    if (tiles * P.N > 0x7fffffffLL) return false;
    P.tiles = (int)tiles;
    return true;
}

// Raises a kernel's dynamic LDS limit; the runtime is asked only when a kernel needs more than it
// was last granted on the current device.
int raise_lds_limit(const void* kern, size_t lds) {
    static std::mutex lock;
    static std::map<std::pair<int, const void*>, size_t> granted;
    int dev = 0;
    if (device_info(nullptr, &dev) != DCN_OK) return DCN_E_DEVICE;
    std::lock_guard<std::mutex> guard(lock);
    size_t& have = granted[std::make_pair(dev, kern)];
    if (lds <= have) return DCN_OK;
    if (hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
        (void)hipGetLastError();
        return fail(DCN_E_LAUNCH, "cannot raise the dynamic LDS limit");
    }
    have = lds;
    return DCN_OK;
}

// Workgroups of a kernel that the current device holds at once (one per CU if the query fails).
long long resident_workgroups(const void* kern, int threads, size_t lds) {
    static std::mutex lock;
    static std::map<std::pair<const void*, size_t>, int> per_cu_of;
    int per_cu = 0;
    {
        std::lock_guard<std::mutex> guard(lock);
        int& v = per_cu_of[std::make_pair(kern, lds)];
        if (v == 0) {
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&v, kern, threads, lds) != hipSuccess || v < 1) {
                (void)hipGetLastError();
                v = 1;
            }
        }
        per_cu = v;
    }
    return (long long)per_cu * cu_count();
}

static HaloPlan halo_plan_of(const Params& P) {
    HaloPlan h;
    for (int a = 0; a < 3; ++a) { h.hext[a] = P.hext[a]; h.mlo[a] = P.mlo[a]; }
    h.hvol = P.hvol; h.hstride = P.hstride; h.cchunk = P.cchunk;
    return h;
}
static bool same_blocks(const Params& a, const Params& b) {
    for (int x = 0; x < 3; ++x)
        if (a.tdim[x] != b.tdim[x] || a.ntile[x] != b.ntile[x]) return false;
    return a.tiles == b.tiles;
}

template <typename K, typename... Args>
int launch_halo(K kern, const char* name, dim3 grid, int threads, size_t lds, hipStream_t s, Args... args) {
    if (lds > 48 * 1024)
        if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kern), lds)) return rc;
    hipLaunchKernelGGL(kern, grid, dim3(threads), lds, s, args...);
    return check_launch(name);
}

// S = T: the float32 / float64 operator.  S = Bf16 / Fp16 (T = float): the tensors are in that
// storage format and only the LDS-halo kernel serves them; where it cannot (halo too large, a layer
// that wants the input-channel split), *declined is set and nothing is launched: the caller then
// widens the tensors and runs the float32 operator.
template <typename T, int ND, typename S = T>
int forward(const Geometry& g, const S* in, const S* w, const S* off, const S* bias, S* out, void* ws,
            size_t ws_bytes, hipStream_t s, bool* declined = nullptr) {
    constexpr bool S16 = !std::is_same<S, T>::value;
    Params P;
    if (int rc = validate(g, P)) return rc;
    if (!in || !w || !off || !out) return fail(DCN_E_ARGUMENT, "null tensor pointer");
    if (int rc = device_info(nullptr)) return rc;
    int MT;
    fwd_weight_pad<T>(P.M, P.Cg, MT, P.mchunks, P.Mp, P.Cgp);
    if (!ws || (!S16 && ws_bytes < (size_t)P.G * P.kV * P.Mp * P.Cgp * sizeof(T))) return fail(DCN_E_WORKSPACE, "workspace too small");
    S* wt = static_cast<S*>(ws);
    const int TN = Mma<T>::TN;
    // Too few position blocks to give every CU a workgroup.  First the input channels of a block are
    // split over up to FWD_MAX_SPLIT workgroups (each samples its own channels once; their partial
    // outputs are joined by a second kernel), as far as the workspace holds the partial outputs.
    // Then fewer row tiles per wavefront: more output-channel chunks, each sampling for itself.
    int fsplit = 1;
    const int mtiles_all = (P.M + TN - 1) / TN;
    const size_t out_bytes = (size_t)P.N * P.C_out * P.outV * sizeof(T);
    const size_t wq_bound = align256(((size_t)chunk_slot<FQ>(P.cpg, P.Cg, P.C_in - 1) + 1) *
                                     forward_slab_elems<T>(P.kV, (mtiles_all + 7) / 8 * 8 * TN) * sizeof(T));
    {
        Params Pt = P;
        const bool tiled = plan_halo<T, ND>(Pt, 144 * 1024, default_margin(), 1 << 30, sizeof(T), WAVESH, false, FQ);
        const long long tiles = tiled ? (long long)Pt.N * Pt.tiles : (long long)P.N * ((P.outV + WAVES * TN - 1) / (WAVES * TN));
        // (eight row tiles per wavefront only pay when the grid is full anyway: measured slower than
        // four with twice the sampling)
        if (MT == 8 && tiles * P.G * P.mchunks < cu_count()) {
            MT = 4;
            P.mchunks = (mtiles_all + MT - 1) / MT;
        }
        if (!S16 && tiled && forward_split() > 1 && (size_t)P.N * P.outV < FWD_SPLIT_POSITIONS && ws_bytes > wq_bound) {
            const size_t room = ws_bytes - wq_bound < FWD_PARTIAL_CAP ? ws_bytes - wq_bound : FWD_PARTIAL_CAP;
            while (fsplit * 2 <= FWD_MAX_SPLIT && fsplit * 2 <= forward_split() && tiles * P.G * P.mchunks * fsplit * 2 <= cu_count() &&
                   (size_t)fsplit * 2 * out_bytes <= room && fsplit * 2 * 16 <= P.Cg)      // at least 16 channels per part
                fsplit *= 2;
        }
        while (MT > 1 && tiles * P.G * P.mchunks * fsplit < cu_count()) {
            MT /= 2;
            P.mchunks = (mtiles_all + MT - 1) / MT;
        }
        P.Mp = P.mchunks * MT * TN;
    }
    // Halo kernel: four channels of a voxel side by side in LDS (forward_quad_kernel).  Few
    // accumulators (MT <= 2): one 1024-thread workgroup per CU with the whole LDS, if its larger halo
    // fits and leaves 8 channels per pass.  Otherwise 512 threads: two workgroups per CU when that
    // still leaves 8 channels per LDS pass, else one large one.  Returns the wavefronts per
    // workgroup, 0 when no halo of margin m fits.
    auto plan_for = [&](int m, Params& Ph) {
        Ph = P;
        int nw = 0;
        // (the 3-D double instance of the 1024-thread shape does not fit its 128 registers)
        if (MT <= 2 && wide_forward() && !(sizeof(T) == 8 && ND == 3)) {
            Params Pw = P;
            if (plan_halo<T, ND>(Pw, 144 * 1024, m, 1 << 30, sizeof(T), 16, false, FQ) &&
                (long long)Pw.N * Pw.tiles * Pw.G * Pw.mchunks <= 0x7fffffffLL &&
                (wide_forward() == 2 || (Pw.cchunk >= 8 && (long long)Pw.N * Pw.tiles * Pw.G * Pw.mchunks >= cu_count()))) {
                Ph = Pw;
                nw = 16;
            }
        }
        if (!nw) {
            bool tiled = plan_halo<T, ND>(Ph, LDS_BUDGET, m, 1 << 30, sizeof(T), WAVESH, false, FQ);
            if ((!tiled || Ph.cchunk < 8) && LDS_BUDGET < 144 * 1024)
                tiled = plan_halo<T, ND>(Ph, 144 * 1024, m, 1 << 30, sizeof(T), WAVESH, false, FQ) || tiled;
            if (!tiled || Ph.cchunk < 8) {       // strided layers: the block shape with the smallest halo may hold 8 channels
                Params Ps = P;
                if (plan_halo<T, ND>(Ps, 144 * 1024, m, 1 << 30, sizeof(T), WAVESH, true, FQ) && (!tiled || Ps.cchunk > Ph.cchunk)) {
                    Ph = Ps;
                    tiled = true;
                }
            }
            if (tiled && (long long)Ph.N * Ph.tiles * Ph.G * Ph.mchunks <= 0x7fffffffLL) nw = WAVESH;
        }
        return nw;
    };
    {
        int margins[MAX_PLANS];
        const int nmargins = plan_margins(ND, margins);
        Params plans[MAX_PLANS];
        const int nw = plan_for(margins[0], plans[0]);
        const size_t slabs = (size_t)chunk_slot<FQ>(P.cpg, P.Cg, P.C_in - 1) + 1;
        const size_t wq_bytes = slabs * forward_slab_elems<T>(P.kV, P.Mp) * sizeof(S);
        if (nw == 16 || ws_bytes < align256(wq_bytes) + (size_t)fsplit * out_bytes) fsplit = 1;
        if (nw && ws_bytes >= wq_bytes) {
            // channels per LDS pass such that every workgroup of a block gets the same number of passes
            auto even_passes = [&](Params& Ph) {
                auto chunks_of_group0 = [&](int cc) {
                    int n = 0;
                    for (int dg = 0; dg <= (P.Cg - 1) / P.cpg; ++dg) {
                        const int len = (P.Cg < (dg + 1) * P.cpg ? P.Cg : (dg + 1) * P.cpg) - dg * P.cpg;
                        n += (len + cc - 1) / cc;
                    }
                    return n;
                };
                for (int cc = Ph.cchunk; cc >= FQ; cc -= FQ)
                    if (chunks_of_group0(cc) % fsplit == 0) { Ph.cchunk = cc; break; }
            };
            if (fsplit > 1) even_passes(plans[0]);
            // Wider halos that one launch of the same kernel can serve as well (same workgroup shape and
            // position blocks); the choice among them is made on the device, see PlanChoice.  The
            // chosen index lives in the last 256 bytes of the workspace.
            PlanChoice pc = {};
            pc.nplans = 1;
            pc.nd = ND;
            pc.margin[0] = margins[0];
            pc.base[0] = 1.f;
            // a wavefront with a sample beyond the halo walks every channel of the pass once more, and each
            // such sample gathers its corners from global memory (fitted to timings at c4 and c3)
            pc.far_wave = ND == 3 ? 0.5f : 0.1f;
            pc.far_sample = ND == 3 ? 2.2f : 5.f;
            const size_t used = align256(wq_bytes) + (fsplit > 1 ? (size_t)fsplit * out_bytes : 0);
            if (nmargins > 1 && ws_bytes >= used + 512) {
                // (within the LDS of the first plan, which fixes how many workgroups share a CU; all of it
                // when the grid gives a CU one workgroup at most)
                const long long wgs = (long long)plans[0].N * plans[0].tiles * plans[0].G * plans[0].mchunks * fsplit;
                size_t lds0 = (size_t)plans[0].cchunk * plans[0].hstride * sizeof(T) + (size_t)plans[0].hvol * 4;
                if (wgs <= cu_count() && lds0 < 144 * 1024) lds0 = 144 * 1024;
                for (int k = 1; k < nmargins; ++k) {
                    Params& Pk = plans[pc.nplans];
                    Pk = P;
                    if (!plan_halo<T, ND>(Pk, lds0, margins[k], 1 << 30, sizeof(T), nw, false, FQ, plans[0].tdim)) continue;
                    if (!same_blocks(Pk, plans[0]) || Pk.hvol > 3 * plans[0].hvol) continue;
                    if (fsplit > 1) even_passes(Pk);
                    pc.margin[pc.nplans] = margins[k];
                    // staging and the per-pass geometry grow with the halo: about a third of the kernel's time in 3-D, an eighth in 2-D
                    pc.base[pc.nplans] = 1.f + (ND == 3 ? 0.3f : 0.12f) * ((float)Pk.hvol / (float)plans[0].hvol - 1.f);
                    ++pc.nplans;
                }
                if (pc.nplans > 1) pc.sel = reinterpret_cast<unsigned*>(static_cast<char*>(ws) + (ws_bytes - 256) / 256 * 256);
            }
            for (int k = pc.nplans; k < MAX_PLANS; ++k) {
                plans[k] = plans[0];
                pc.margin[k] = pc.margin[pc.nplans - 1];
                pc.base[k] = 1e30f;
            }
            PlanSet alts;
            for (int k = 1; k < MAX_PLANS; ++k) alts.alt[k - 1] = halo_plan_of(plans[k]);
            alts.mask = (1u << pc.nplans) - 1;
            {
                const size_t total = (size_t)chunk_candidates<FQ>(P.cpg, P.Cg, P.C_in) * forward_slab_elems<T>(P.kV, P.Mp);
                const unsigned blocks = (unsigned)((total + 255) / 256 > 8192 ? 8192 : (total + 255) / 256);
                const size_t n_off = (size_t)P.N * P.DG * P.kV * ND * P.outV;
                hipLaunchKernelGGL((pack_forward_weight_kernel<T, S>), dim3(blocks + (pc.sel ? 1 : 0)), dim3(256), 0, s, plans[0], w, wt, pc, off, n_off);
                if (int rc = check_launch("pack_forward_weight_kernel")) return rc;
            }
            size_t lds = 0;
            for (int k = 0; k < pc.nplans; ++k) {
                const size_t l = (size_t)plans[k].cchunk * plans[k].hstride * sizeof(T) + (size_t)plans[k].hvol * 4;
                if (l > lds) lds = l;
            }
            const Params& Ph = plans[0];
            using Kern = void (*)(Params, PlanSet, const unsigned*, const S*, const S*, const S*, const S*, S*, T*, int, unsigned, TailSplit);
            Kern kern;
            if (nw == 16) kern = MT == 1 ? forward_quad_kernel<T, ND, 1, 16, S> : forward_quad_kernel<T, ND, 2, 16, S>;
            else kern = MT == 1 ? forward_quad_kernel<T, ND, 1, WAVESH, S> : MT == 2 ? forward_quad_kernel<T, ND, 2, WAVESH, S>
                      : MT == 4 ? forward_quad_kernel<T, ND, 4, WAVESH, S> : forward_quad_kernel<T, ND, 8, WAVESH, S>;
            T* part = reinterpret_cast<T*>(static_cast<char*>(ws) + align256(wq_bytes));      // partial sums, in the arithmetic type
            // A grid that ends in a partly filled round of workgroups: the units of that round, last in
            // the launch, are split over several workgroups each (every tsplit-th channel pass), so that
            // the round fills the device; forward_join_tail_kernel adds their partial sums.  Either all
            // of them tsplit ways, or -- when that leaves the last of the resulting short rounds partly
            // empty -- as many of them tsplit + 1 ways as make the workgroup count a whole number of
            // rounds (TailSplit: the units split tsplit ways come first, so that the longer workgroups
            // start first).  Cost of a workgroup: per channel pass one part for the tap geometry and one
            // per four channels, plus 5 % of a unit for its fixed part (halo table, offsets, output).
            const long long units = (long long)Ph.N * Ph.tiles * Ph.G * Ph.mchunks;
            int tsplit = 1;
            long long whole = 0;
            TailSplit ts = {0u, 0, 0};
            if (fsplit == 1 && forward_tail_split()) {
                const long long slots = forward_slots() ? forward_slots() : resident_workgroups(reinterpret_cast<const void*>(kern), nw * 64, lds);
                const long long rest = units % slots;
                constexpr double GEO = 0.45;    // tap geometry of a pass, in units of four channels' sampling and contraction
                // cost of the longest workgroup when the passes of a unit (cch channels each) are dealt to cs workgroups
                auto wg_cost = [&](int cs, int cch, int* npasses) {
                    double load[64] = {0};
                    int k = 0;
                    for (int dg = 0; dg <= (P.Cg - 1) / P.cpg; ++dg) {
                        const int len = (P.Cg < (dg + 1) * P.cpg ? P.Cg : (dg + 1) * P.cpg) - dg * P.cpg;
                        for (int c0 = 0; c0 < len; c0 += cch, ++k) load[k % cs] += GEO + (double)(((len - c0 < cch ? len - c0 : cch) + FQ - 1) / FQ);
                    }
                    if (npasses) *npasses = k;
                    double worst = 0;
                    for (int z = 0; z < cs; ++z) worst = load[z] > worst ? load[z] : worst;
                    return worst;
                };
                int passes = 0;                 // channel passes of a unit under the first plan
                const double unit_cost = wg_cost(1, Ph.cchunk, &passes);
                const size_t end = pc.sel ? (ws_bytes - 256) / 256 * 256 : ws_bytes;
                const size_t room = end > align256(wq_bytes) ? end - align256(wq_bytes) : 0;
                const size_t per_wg = (size_t)MT * TN * nw * TN * sizeof(T);
                if (units > slots && rest) {
                    double best = 0.9;          // of the time of an unsplit last round; a tenth must be gained
                    for (int cs = 2; cs <= 8 && cs <= passes; ++cs) {
                        if (forward_tail_split() > 1 && cs != forward_tail_split()) continue;
                        const long long rounds = (rest * cs + slots - 1) / slots;
                        const double ta = wg_cost(cs, Ph.cchunk, nullptr) / unit_cost + 0.05;
                        {
                            const double t = (double)rounds * ta;
                            const size_t bytes = (size_t)rest * cs * per_wg;
                            if ((t < best || forward_tail_split() > 1) && bytes <= room && bytes <= FWD_PARTIAL_CAP) {
                                best = t; tsplit = cs; ts = TailSplit{0u, 0, 0};
                            }
                        }
                        // two runs: nb units cs + 1 ways, the others cs ways, rounds * slots workgroups in all;
                        // the cs-way workgroups must fit the first round
                        const long long nb = rounds * slots - rest * cs;
                        if (!forward_tail_two_runs() || cs + 1 > 8 || nb <= 0 || nb >= rest || (rest - nb) * cs > slots) continue;
                        double tb = 1e30;
                        int cchb = Ph.cchunk;
                        for (int cch = Ph.cchunk; cch >= FQ; cch -= FQ) {
                            int np = 0;
                            const double c = wg_cost(cs + 1, cch, &np) / unit_cost + 0.05;
                            if (np >= cs + 1 && c < tb) { tb = c; cchb = cch; }
                        }
                        const double t = ta + (double)(rounds - 1) * tb;
                        const size_t bytes = (size_t)(rounds * slots) * per_wg;
                        if (t < best && bytes <= room && bytes <= FWD_PARTIAL_CAP) {
                            best = t; tsplit = cs; ts = TailSplit{(unsigned)(rest - nb), cs + 1, cchb};
                        }
                    }
                    if (tsplit > 1) whole = units - rest;
                }
            }
            const long long wgs = tsplit > 1 ? whole + (ts.splitB ? (long long)ts.unitsA * tsplit + (units - whole - ts.unitsA) * ts.splitB : (units - whole) * tsplit)
                                             : units * fsplit;
            if (wgs > 0x7fffffffLL) return fail(DCN_E_ARGUMENT, "too many workgroups for one launch");
            const dim3 grid((unsigned)wgs);
            if (trace_plans()) {
                fprintf(stderr, "dcn forward: %d wavefronts, MT %d, grid %u (%lld unsplit, rest x %d), LDS %zu, every unit split x %d\n", nw, MT, grid.x,
                        tsplit > 1 ? whole : 0LL, tsplit, lds, fsplit);
                if (ts.splitB) fprintf(stderr, "  of the rest: %u units x %d, the others x %d with %d channels per pass\n", ts.unitsA, tsplit, ts.splitB, ts.cchB);
                for (int k = 0; k < pc.nplans; ++k)
                    fprintf(stderr, "  plan %d: margin %d, halo %d x %d x %d, %d channels per pass, base cost %.3f\n", k, pc.margin[k],
                            plans[k].hext[0], plans[k].hext[1], plans[k].hext[2], plans[k].cchunk, pc.base[k]);
            }
            const unsigned* sel = pc.sel;
            if (int rc = launch_halo(kern, "forward_quad_kernel", grid, nw * 64, lds, s, Ph, alts, sel, in, off, (const S*)wt, bias, out, part,
                                     tsplit > 1 ? tsplit : fsplit, (unsigned)whole, ts))
                return rc;
            if (fsplit == 1 && tsplit == 1) return DCN_OK;
            if (tsplit > 1) {
                using Join = void (*)(Params, PlanSet, const unsigned*, const T*, const S*, S*, int, unsigned, TailSplit);
                Join join;
                if (nw == 16) join = MT == 1 ? forward_join_tail_kernel<T, ND, 1, 16, S> : forward_join_tail_kernel<T, ND, 2, 16, S>;
                else join = MT == 1 ? forward_join_tail_kernel<T, ND, 1, WAVESH, S> : MT == 2 ? forward_join_tail_kernel<T, ND, 2, WAVESH, S>
                          : MT == 4 ? forward_join_tail_kernel<T, ND, 4, WAVESH, S> : forward_join_tail_kernel<T, ND, 8, WAVESH, S>;
                hipLaunchKernelGGL(join, dim3((unsigned)((units - whole) * (MT * TN / JOIN_ROWS))), dim3(nw * TN), 0, s, Ph, alts, sel, (const T*)part, bias, out, tsplit, (unsigned)whole, ts);
                return check_launch("forward_join_tail_kernel");
            }
            if constexpr (!S16) {
                const size_t total = (size_t)P.N * P.C_out * P.outV;
                const unsigned jb = (unsigned)((total + 255) / 256 > 4096 ? 4096 : (total + 255) / 256);
                hipLaunchKernelGGL(forward_join_partials_kernel<T>, dim3(jb), dim3(256), 0, s, part, bias, out, fsplit, total, P.C_out, P.outV);
                return check_launch("forward_join_partials_kernel");
            }
        }
    }
    if constexpr (S16) {
        if (declined) *declined = true;
        return DCN_OK;
    } else {
    if (int rc = relayout<T>(P, w, wt, 0, s)) return rc;
    // geometry whose halo does not fit in LDS: gather straight from global memory
    P.tiles = (P.outV + WAVES * TN - 1) / (WAVES * TN);
    if ((long long)P.N * P.tiles > 0x7fffffffLL || (long long)P.G * P.mchunks > 65535)
        return fail(DCN_E_ARGUMENT, "layer too large for the kernel without LDS tiling (groups x output-channel chunks > 65535)");
    const dim3 grid((unsigned)P.N * P.tiles, (unsigned)P.G * P.mchunks);
    switch (MT) {
        case 1: hipLaunchKernelGGL((forward_kernel<T, ND, 1>), grid, dim3(WG), 0, s, P, in, off, wt, bias, out); break;
        case 2: hipLaunchKernelGGL((forward_kernel<T, ND, 2>), grid, dim3(WG), 0, s, P, in, off, wt, bias, out); break;
        case 4: hipLaunchKernelGGL((forward_kernel<T, ND, 4>), grid, dim3(WG), 0, s, P, in, off, wt, bias, out); break;
        default: hipLaunchKernelGGL((forward_kernel<T, ND, 8>), grid, dim3(WG), 0, s, P, in, off, wt, bias, out); break;
    }
    return check_launch("forward_kernel");
    }
}

template <typename T>
int absmax(const T* w, size_t n, float* out, hipStream_t s) {
    hipLaunchKernelGGL(fill_zero_kernel<float>, dim3(1), dim3(64), 0, s, out, (size_t)1);
    if (int rc = check_launch("fill_zero_kernel")) return rc;
    const unsigned blocks = (unsigned)((n + 1023) / 1024 > 128 ? 128 : (n + 1023) / 1024);
    hipLaunchKernelGGL(absmax_kernel<T>, dim3(blocks ? blocks : 1), dim3(256), 0, s, w, n, out);
    return check_launch("absmax_kernel");
}
// out[0] = max |w|, out[1] = largest norm over the output channels of a group of an (input channel, tap)
// column; `out` was cleared by the pack_weight_kernel launched before
template <typename T>
int weight_bounds(const Params& P, const T* w, float* out, hipStream_t s) {
    const size_t cols = (size_t)P.Cg * P.kV;
    if (P.G > 65535) return fail(DCN_E_ARGUMENT, "more than 65535 convolution groups");
    hipLaunchKernelGGL(weight_bounds_kernel<T>, dim3((unsigned)((cols + 63) / 64), (unsigned)P.G), dim3(512), 0, s, w, P.M, cols, out);
    return check_launch("weight_bounds_kernel");
}

constexpr unsigned FLAG_INPUT_ONLY = 0x100u;     // internal: see backward_input_offset
// S = T: the float32 / float64 operator.  S = Bf16 / Fp16 (T = float): input, weight, offset and
// grad_output are in that storage format (the gradients are float), and only the fused kernel with
// its grad_output operand in registers serves them, on the 16-bit matrix instructions; where it
// cannot, *declined is set and nothing is launched: the caller then widens the tensors and runs the
// float32 operator.
template <typename T, int ND, typename S = T>
int backward_input_offset(const Geometry& g, const S* in, const S* w, const S* off, const S* gout, T* gin,
                          T* goff, void* ws, size_t ws_bytes, hipStream_t s, unsigned flags = 0, bool* declined = nullptr) {
    constexpr bool S16 = !std::is_same<S, T>::value;
    Params P;
    if (int rc = validate(g, P)) return rc;
    if (flags & ~(unsigned)(DCN_FLAG_OOB_OFFSET_GRAD_ZERO | FLAG_INPUT_ONLY)) return fail(DCN_E_ARGUMENT, "unknown flag");
    if (int rc = device_info(nullptr)) return rc;
    P.oob_zero = (flags & DCN_FLAG_OOB_OFFSET_GRAD_ZERO) ? 1 : 0;
    // grad_input alone (the plain convolution's backward-to-input, which is not given the input): the
    // scatter kernels need no input values; `goff` is then scratch for the one kernel that writes it anyway
    const bool input_only = (flags & FLAG_INPUT_ONLY) != 0;
    if ((!in && !input_only) || !w || !off || !gout || !gin || !goff) return fail(DCN_E_ARGUMENT, "null tensor pointer");
    bwd_data_weight_pad<T>(P.M, P.Cg, P.Mp, P.Cgp);
    const size_t wbytes = bwd_data_weight_bytes<T>(P.M, P.Cg, P.kV, P.G, P.cpg);
    const size_t tbytes = align256((size_t)P.N * P.C_in * P.inV * sizeof(T));
    if (!ws || ws_bytes < wbytes + 2 * tbytes) return fail(DCN_E_WORKSPACE, "workspace too small");
    S* wt = static_cast<S*>(ws);
    T* in_cl = reinterpret_cast<T*>(static_cast<char*>(ws) + wbytes);
    T* gin_cl = reinterpret_cast<T*>(static_cast<char*>(ws) + wbytes + tbytes);
    const int TN = Mma<T>::TN;
    const int mk = bwd_data_mk<T>(P.M);
    // weight bounds (two floats) and, 64 bytes further, the plan chosen on the device: in the last whole
    // 256-byte block of the workspace when that lies behind the two channels-last regions
    // (dcn_workspace_bytes counts it), else at the start of the channels-last gradient, which the LDS
    // paths do not use
    const size_t tail_at = ws_bytes >= 256 ? (ws_bytes - 256) / 256 * 256 : 0;
    const bool tail_words = tail_at >= wbytes + 2 * tbytes;
    float* wmax = tail_words ? reinterpret_cast<float*>(static_cast<char*>(ws) + tail_at) : reinterpret_cast<float*>(gin_cl);
    const dim3 tgrid((P.inV + 31) / 32, (unsigned)(P.C_in + 31) / 32, (unsigned)P.N), tblock(32, 8);

    // 1) one kernel: scatter privatised in LDS + coordinate gradient from an LDS input halo
    // A halo of up to FUSED_HS cells gets the variant with that compile-time plane stride (the four
    // planes of either kind then lie within the 64 KB reach of an LDS instruction's offset field).
    // Eight wavefronts per workgroup; four (half the positions, in the block shape with the smallest
    // halo) where only that fits, e.g. under stride 2.
    constexpr int FUSED_HS = sizeof(T) == 4 ? 2720 : 2112;
    constexpr int FUSED_HS8 = 2016;     // plane stride of the 8-channel float instantiation with compile-time halo extents
    using Kern = void (*)(Params, PlanSet, const unsigned*, const S*, const S*, const S*, const S*, const float*, T*, T*, int, unsigned, int);
    struct FusedPlan {
        Params Ph;
        Kern kern;
        int nw, cch, csplit, goff_atomic;
        bool zero_goff;
        bool wide;
        long long whole, items, slots;
        size_t lds;
        const S* wt;
    };
    const int seg = P.cpg < P.Cg ? P.cpg : P.Cg;
    // Plans the fused kernel for a halo of margin m; false when none of its shapes fits.
    // (attempts: eight wavefronts on the default block, eight on the block shape with the smallest
    // halo, four on the block shape with the smallest halo)
    auto plan_fused = [&](int m, FusedPlan& fp) {
        for (int attempt = fused_first_waves() == 8 ? 0 : 2; attempt < 3; ++attempt) {
            const int nw = attempt < 2 ? 8 : 4;
            const bool smallest = attempt > 0;
            Params Ph = P;
            // float32: two channels per LDS cell as 32-bit fixed point while the terms one cell can receive
            // (positions of the block x taps) leave at least 17 bits below the largest possible term
            const bool pair = sizeof(T) == 4 && fused_pair() && (long long)nw * TN * P.kV <= (1 << 14);
            const size_t chb = (pair ? 4 : 8) + sizeof(T);      // LDS bytes per channel and halo voxel: cell + input value
            // Channels per chunk: 8 where that takes fewer MFMA passes per channel (a pass holds TN / CCH
            // taps: the 9 taps of a 3x3 kernel are 2 float passes per 4 channels or 3 per 8; the 27 of a
            // 3x3x3 kernel 4 or 7) and the planes of 8 channels fit: the small halos of 2-D layers, and
            // 3-D ones with paired cells.  16 (2-D, float, paired cells): two taps per pass -- the 9 taps of
            // a 3x3 kernel are 5 passes per 16 channels instead of 6.  The float kernel with 8 channels
            // per chunk keeps the input values bank-swizzled and wants the innermost halo extent a
            // multiple of the four-channel groups per voxel.
            auto passes = [&](int c) { const int tp = Mma<T>::TN / c; return (P.kV + tp - 1) / tp; };
            int cch = 0;
            size_t tables = 0;
            bool fixed = false, special = false;
            for (int cand = 16; cand >= 4 && !cch; cand /= 2) {
                if (cand >= 8 && !((ND == 2 || pair) && nw == 8 && fused_chunk8() && seg >= 8 && passes(8) * 4 < passes(4) * 8)) continue;
                if (cand == 16 && !(ND == 2 && pair && fused_chunk16() && seg >= 16 && passes(16) * 8 < passes(8) * 16)) continue;
                Params Pc = P;
                const int wmult = cand == 16 ? 1 : cand == 8 ? swizzle_groups<T, 8>() : 1;
                if (!plan_halo<T, ND>(Pc, scatter_budget(), m, 8, chb, nw, smallest, 0, nullptr, wmult)) continue;
                const size_t tb = (size_t)Pc.hvol * 4;      // halo table
                if ((long long)Pc.N * Pc.tiles * Pc.DG * 4 > 0x7fffffffLL) continue;
                if (cand >= 8) {
                    if ((scatter_budget() - tb) / ((size_t)Pc.hstride * chb) < (size_t)cand) continue;
                } else {
                    // A halo of up to FUSED_HS cells gets the variant with that compile-time plane stride
                    fixed = fused_fixed_stride() && Pc.hvol <= FUSED_HS && (size_t)4 * FUSED_HS * chb + tb <= scatter_budget();
                    if (!fixed && (scatter_budget() - tb) / ((size_t)Pc.hstride * chb) < 4) continue;
                }
                Ph = Pc;
                tables = tb;
                cch = cand;
            }
            if (!cch) continue;
            const bool sixteen = cch == 16, eight = cch >= 8;
            Ph.cchunk = cch;
            if (fixed && !eight) Ph.hstride = FUSED_HS;
            // grad_output operand held in registers when its reduction steps fit: 32 per pass
            // (M <= 64 float, 128 double with 4-channel chunks)
            // (16-bit storage: a reduction step takes 8 output channels and an operand batch half as many steps)
            const int KS = GcolGemm<T, S>::KS, halve = S16 ? 2 : 1;
            const int ksteps = (P.M + KS - 1) / KS;
            const bool wide = eight && !sixteen && pair && ksteps <= 32 / halve;                     // the kernel's WIDE
            const int slot_regs = (wide || sixteen) ? 8 : (Mma<T>::row(1, 0) - Mma<T>::row(0, 0) == 1) ? 4 : cch / 4;      // the kernel's RPS
            const bool breg = ksteps <= Mma<T>::NACC / slot_regs * ((wide || sixteen) ? 16 : 8) / halve;
            // float, 4-channel chunks: a second set of 32 registers takes the operand of up to 128 output channels (16-bit: 256)
            const bool breg2 = sizeof(T) == 4 && !eight && !breg && ksteps <= 64 / halve && fused_breg2();
            special = ND == 3 && eight && !sixteen && pair && wide && breg && fused_fixed_stride() && Ph.hext[1] == 14 && Ph.hext[2] == 14 &&
                      Ph.hstride <= FUSED_HS8;
            if (special) Ph.hstride = FUSED_HS8;
            const size_t lds = (size_t)cch * Ph.hstride * chb + tables;
            Kern kern = nullptr;
#define DCN_FUSED_C(CCH_, BREG_, HS_, NW_, PAIR_) backward_input_halo_kernel<T, ND, CCH_, true, (BREG_) || S16, HS_, NW_, true, PAIR_, 1, 0, 0, S>
#define DCN_FUSED_B2(HS_, NW_, PAIR_) backward_input_halo_kernel<T, ND, 4, true, true, HS_, NW_, true, PAIR_, 2, 0, 0, S>
            auto pick = [&](auto pair_tag) {
                constexpr bool PR = decltype(pair_tag)::value;
                if (sixteen) {
                    if constexpr (ND == 2 && PR && sizeof(T) == 4) kern = breg ? DCN_FUSED_C(16, true, 0, 8, PR) : DCN_FUSED_C(16, false, 0, 8, PR);
                } else if (eight) {
                    if constexpr (ND == 2 || PR) kern = breg ? DCN_FUSED_C(8, true, 0, 8, PR) : DCN_FUSED_C(8, false, 0, 8, PR);
                    // the halo of a 3x3x3 kernel at stride 1 and margin 2 under the default block of positions:
                    // inner extents 14 x 14 and the plane stride fixed at compile time
                    if constexpr (ND == 3 && PR && sizeof(T) == 4) {
                        if (special) kern = backward_input_halo_kernel<T, ND, 8, true, true, FUSED_HS8, 8, true, true, 1, 14, 14, S>;
                    }
                } else if (breg2) {
                    if constexpr (sizeof(T) == 4) {
                        if (nw == 8) kern = fixed ? DCN_FUSED_B2(FUSED_HS, 8, PR) : DCN_FUSED_B2(0, 8, PR);
                        else kern = fixed ? DCN_FUSED_B2(FUSED_HS, 4, PR) : DCN_FUSED_B2(0, 4, PR);
                    }
                } else if (nw == 8)
                    kern = fixed && breg ? DCN_FUSED_C(4, true, FUSED_HS, 8, PR) : fixed ? DCN_FUSED_C(4, false, FUSED_HS, 8, PR) : DCN_FUSED_C(4, false, 0, 8, PR);
                else
                    kern = fixed && breg ? DCN_FUSED_C(4, true, FUSED_HS, 4, PR) : fixed ? DCN_FUSED_C(4, false, FUSED_HS, 4, PR) : DCN_FUSED_C(4, false, 0, 4, PR);
            };
            if constexpr (sizeof(T) == 4) {
                if (pair) pick(std::true_type{});
                else pick(std::false_type{});
            } else
                pick(std::false_type{});
#undef DCN_FUSED_B2
#undef DCN_FUSED_C
            if (!kern) continue;
            if (S16 && !breg && !breg2) continue;       // 16-bit operands come from registers only
            // Work items are (tile, deformable group) pairs, each a run of nchunks channel chunks.  `slots`
            // workgroups run at once, so the items take whole rounds plus a partly filled last one.  Either
            // every item is split over 1, 2 or 4 workgroups (workgroup cz takes every csplit-th chunk), or
            // the items of the whole rounds stay unsplit and only those of the last round are split, as
            // finely as fills the device; they come last in the launch.  A workgroup's fixed part
            // (grad_output operand, halo table, offsets) costs about a quarter of a chunk, which the
            // estimate charges per split.  The workgroups that share an item add their grad_offset parts with
            // float atomics on a zero-filled buffer; the only owner of an item stores running sums.
            const int nchunks = (seg + cch - 1) / cch;
            const long long items = (long long)Ph.N * Ph.tiles * Ph.DG;
            const long long slots = forced_slots() ? forced_slots() : resident_workgroups(reinterpret_cast<const void*>(kern), nw * 64, lds);
            auto item_cost = [&](double chunks_per_wg, int wgs) { return wgs * (chunks_per_wg + 0.25) / nchunks; };
            int csplit = 1;
            long long whole = 0;                              // unsplit items at the start of the launch
            double best = 1e30;
            for (int cs = 1; cs <= 4 && cs <= nchunks; cs *= 2) {
                const double rounds = (double)((items * cs + slots - 1) / slots) / cs * item_cost((double)nchunks / cs, cs);
                if (rounds < best) { best = rounds; csplit = cs; }
            }
            if (fused_tail_split() && items > slots && items % slots) {
                const long long rest = items % slots;
                const long long cs = slots / rest < nchunks ? slots / rest : nchunks;
                if (cs >= 2) {
                    const double rounds = (double)(items / slots) * item_cost(nchunks, 1) + item_cost((double)((nchunks + cs - 1) / cs), 1);
                    if (rounds < best) { best = rounds; csplit = (int)cs; whole = items - rest; }
                }
            }
            if (forced_csplit()) { csplit = forced_csplit(); whole = 0; }
            if (csplit > nchunks) csplit = nchunks;
            if (whole + (items - whole) * csplit > 0x7fffffffLL) continue;
            fp.Ph = Ph; fp.kern = kern; fp.nw = nw; fp.cch = cch; fp.csplit = csplit;
            // grad_offset over the chunks of an item that one workgroup owns: the running sum through plain
            // loads and stores in the 3-D kernels (float atomics run at about 3e11 per second over the device,
            // and a 3x3x3 layer has 81 grad_offset elements per position and chunk); atomics in the 2-D ones
            fp.goff_atomic = ND == 2 && nchunks > 1 ? 1 : 0;
            fp.zero_goff = fp.goff_atomic || csplit > 1;
            fp.wide = wide; fp.whole = whole; fp.items = items; fp.slots = slots; fp.lds = lds; fp.wt = nullptr;
            return true;
        }
        return false;
    };
    FusedPlan fp[MAX_PLANS];
    int margins[MAX_PLANS];
    const int nmargins = plan_margins(ND, margins);
    if (S16 && !(scatter_in_lds() && fused_coord() && !input_only && native16())) {
        if (declined) *declined = true;
        return DCN_OK;
    }
    if (scatter_in_lds() && fused_coord() && !input_only && plan_fused(margins[0], fp[0])) {
        // Wider halos for offsets that reach further; the choice is made on the device, see
        // PlanChoice.  A plan whose weights want another lane order gets a packed copy of its own in
        // the region of the channels-last input, which this path does not use.
        PlanChoice pc = {};
        pc.nplans = 1;
        pc.nd = ND;
        pc.margin[0] = margins[0];
        pc.base[0] = 1.f;
        pc.far_sample = ND == 3 ? 4.5f : 1.f;       // a sample beyond the halo scatters with global atomics
        pc.far_steep = ND == 3 ? 25.f : 0.f;        // (c4, margin 2: 3.0, 4.1, 10.4, 26.6 times the time at 49, 70, 87.5, 96 % of the samples beyond the halo)
        // 3-D: when most samples leave even the widest halo, the path without LDS tiling (coalesced
        // atomics on a channels-last copy; about 6.5 times the fused kernel's time on small offsets,
        // whatever the offsets) is the cheaper one: offered as a fourth choice, its kernels launched
        // behind the fused ones and gated on the choice (DCN_GLOBAL_PLAN=0: not offered)
        const bool offer_global = !S16 && ND == 3 && tail_words && global_plan() && (long long)P.N * ((P.outV + WAVES * TN - 1) / (WAVES * TN)) <= 0x7fffffffLL &&
                                  P.DG <= 65535;
        int copies = 1;                             // packed weight copies
        fp[0].wt = wt;
        for (int k = 1; k < nmargins; ++k) {
            FusedPlan& c = fp[pc.nplans];
            if (!plan_fused(margins[k], c) || c.Ph.hvol > 3 * fp[0].Ph.hvol) continue;
            for (int e = 0; e < pc.nplans && !c.wt; ++e)
                if (fp[e].cch == c.cch && fp[e].wide == c.wide) c.wt = fp[e].wt;
            if (!c.wt) {
                if ((size_t)copies * wbytes > tbytes) continue;
                c.wt = reinterpret_cast<const S*>(reinterpret_cast<const char*>(in_cl) + (size_t)(copies - 1) * wbytes);
                ++copies;
            }
            pc.margin[pc.nplans] = margins[k];
            // flush, staging and the per-chunk passes grow with the halo: most of the kernel's time in 3-D, little in 2-D
            // (a quarter more where only the shape with half the wavefronts fits)
            pc.base[pc.nplans] = (1.f + (ND == 3 ? 0.9f : 0.05f) * ((float)c.Ph.hvol / (float)fp[0].Ph.hvol - 1.f)) * (c.nw < fp[0].nw ? 1.25f : 1.f);
            ++pc.nplans;
        }
        for (int k = pc.nplans; k < MAX_PLANS; ++k) {
            pc.margin[k] = pc.margin[pc.nplans - 1];
            pc.base[k] = 1e30f;
        }
        unsigned* sel = (pc.nplans > 1 || offer_global) ? reinterpret_cast<unsigned*>(wmax + 16) : nullptr;
        pc.sel = sel;
        pc.global_cost = offer_global ? 6.5f : 0.f;
        const size_t n_off = (size_t)P.N * P.DG * P.kV * ND * P.outV;
        // weights in the lane order of the kernel's operand loads, one slab per channel chunk; the
        // first launch clears the weight bounds and chooses the plan
        for (int k = 0; k < pc.nplans; ++k) {
            bool packed = false;
            for (int e = 0; e < k; ++e) packed = packed || fp[e].wt == fp[k].wt;
            if (packed) continue;
            const bool sixteen = fp[k].cch == 16, eight = fp[k].cch == 8, wide = fp[k].wide;
            const size_t total = packed_weight_elems<T, S>(P.M, P.kV, (size_t)(sixteen ? chunk_candidates<16>(P.cpg, P.Cg, P.C_in)
                                                                            : eight ? chunk_candidates<8>(P.cpg, P.Cg, P.C_in)
                                                                                    : chunk_candidates<4>(P.cpg, P.Cg, P.C_in)), fp[k].cch);
            const unsigned blocks = (unsigned)((total + 255) / 256 > 8192 ? 8192 : (total + 255) / 256);
            PlanChoice pk = pc;
            if (k > 0) pk.sel = nullptr;
            float* bounds = k == 0 ? wmax : nullptr;
            S* dst = const_cast<S*>(fp[k].wt);
            const dim3 pgrid(blocks + (pk.sel ? 1 : 0));
            // (wide: row order that leaves the eight channels of a tap in one lane)
            if (sixteen) hipLaunchKernelGGL((pack_weight_kernel<T, 16, false, S>), pgrid, dim3(256), 0, s, P, w, dst, bounds, pk, off, n_off);
            else if (wide) hipLaunchKernelGGL((pack_weight_kernel<T, 8, true, S>), pgrid, dim3(256), 0, s, P, w, dst, bounds, pk, off, n_off);
            else if (eight) hipLaunchKernelGGL((pack_weight_kernel<T, 8, false, S>), pgrid, dim3(256), 0, s, P, w, dst, bounds, pk, off, n_off);
            else hipLaunchKernelGGL((pack_weight_kernel<T, 4, false, S>), pgrid, dim3(256), 0, s, P, w, dst, bounds, pk, off, n_off);
            if (int rc = check_launch("pack_weight_kernel")) return rc;
        }
        if (int rc = weight_bounds<S>(P, w, wmax, s)) return rc;
        bool any_atomic = false;
        for (int k = 0; k < pc.nplans; ++k) any_atomic = any_atomic || fp[k].zero_goff;
        if (any_atomic) {
            const size_t nel = (size_t)P.N * P.DG * P.kV * ND * P.outV;
            const unsigned fb = (unsigned)((nel + 1023) / 1024 > 8192 ? 8192 : (nel + 1023) / 1024);
            hipLaunchKernelGGL(fill_zero_kernel<T>, dim3(fb), dim3(256), 0, s, goff, nel);
            if (int rc = check_launch("fill_zero_kernel")) return rc;
        }
        // one launch per set of plans that differ in nothing but the halo
        unsigned launched = 0;
        for (int k = 0; k < pc.nplans; ++k) {
            if ((launched >> k) & 1u) continue;
            // (the kernel takes plan 0 as its Params argument: a launch that does not serve plan 0 gets
            // the Params of its first plan there, which its mask never selects as such)
            PlanSet alts;
            alts.mask = 0;
            size_t lds = 0;
            for (int e = 1; e < MAX_PLANS; ++e) alts.alt[e - 1] = halo_plan_of(fp[k].Ph);
            for (int e = k; e < pc.nplans; ++e) {
                const bool same = fp[e].kern == fp[k].kern && fp[e].wt == fp[k].wt && fp[e].csplit == fp[k].csplit && fp[e].whole == fp[k].whole &&
                                  fp[e].items == fp[k].items && fp[e].goff_atomic == fp[k].goff_atomic && fp[e].nw == fp[k].nw &&
                                  fp[e].slots == fp[k].slots && same_blocks(fp[e].Ph, fp[k].Ph);      // (as many workgroups per CU with the larger LDS)
                if (!same) continue;
                if (e > 0) alts.alt[e - 1] = halo_plan_of(fp[e].Ph);
                alts.mask |= 1u << e;
                if (fp[e].lds > lds) lds = fp[e].lds;
            }
            launched |= alts.mask;
            if (trace_plans()) {
                fprintf(stderr, "dcn backward_input_offset: launch for plans %#x: %d wavefronts, %d channels per chunk%s, grid %lld (%lld unsplit, rest x %d), LDS %zu\n",
                        alts.mask, fp[k].nw, fp[k].cch, fp[k].wide ? " (wide)" : "", fp[k].whole + (fp[k].items - fp[k].whole) * fp[k].csplit, fp[k].whole,
                        fp[k].csplit, lds);
                for (int e = 0; e < pc.nplans; ++e)
                    if ((alts.mask >> e) & 1u)
                        fprintf(stderr, "  plan %d: margin %d, halo %d x %d x %d, base cost %.3f\n", e, pc.margin[e], fp[e].Ph.hext[0], fp[e].Ph.hext[1],
                                fp[e].Ph.hext[2], pc.base[e]);
            }
            if (lds > 48 * 1024)
                if (int rc = raise_lds_limit(reinterpret_cast<const void*>(fp[k].kern), lds)) return rc;
            hipLaunchKernelGGL(fp[k].kern, dim3((unsigned)(fp[k].whole + (fp[k].items - fp[k].whole) * fp[k].csplit)), dim3(fp[k].nw * 64), lds, s,
                               fp[k].Ph, alts, (const unsigned*)sel, in, off, fp[k].wt, gout, (const float*)wmax, gin, goff, fp[k].csplit, (unsigned)fp[k].whole,
                               fp[k].goff_atomic);
            if (int rc = check_launch("backward_input_halo_kernel")) return rc;
        }
        if constexpr (!S16) if (offer_global) {
            // the fourth choice: three launches that return at once unless *sel == MAX_PLANS.  They reuse
            // the weight region and the channels-last regions, which the fused kernels no longer read then.
            Params Pg = P;
            Pg.tiles = (P.outV + WAVES * TN - 1) / (WAVES * TN);
            const size_t total_w = (size_t)P.G * P.kV * P.Mp * P.Cgp, pad_w = (size_t)TAP_PAD * P.Mp * P.Cgp;
            const size_t nelem = (size_t)P.N * P.C_in * P.inV;
            const unsigned nb_w = (unsigned)((total_w + pad_w + 255) / 256 > 1024 ? 1024 : (total_w + pad_w + 255) / 256);
            const unsigned nb_z = (unsigned)((nelem + 1023) / 1024 > 4096 ? 4096 : (nelem + 1023) / 1024);
            const size_t ntiles = (size_t)P.N * ((P.C_in + 31) / 32) * ((P.inV + 31) / 32);
            const unsigned nb_t = (unsigned)(ntiles > 16384 ? 16384 : ntiles);
            if (trace_plans()) fprintf(stderr, "dcn backward_input_offset: path without LDS tiling offered at cost %.2f\n", pc.global_cost);
            hipLaunchKernelGGL(global_path_prepare_kernel<T>, dim3(nb_w + nb_z + nb_t), dim3(256), 0, s, Pg, w, wt, pad_w, gin_cl, in, in_cl,
                               nb_w, nb_z, (const unsigned*)sel, (unsigned)MAX_PLANS);
            if (int rc = check_launch("global_path_prepare_kernel")) return rc;
            hipLaunchKernelGGL((backward_data_kernel<T, ND, true, 0>), dim3((unsigned)Pg.N * Pg.tiles, (unsigned)P.DG), dim3(WG), 0, s, Pg,
                               (const T*)in_cl, off, (const T*)wt, gout, gin_cl, goff, (const unsigned*)sel, (unsigned)MAX_PLANS);
            if (int rc = check_launch("backward_data_kernel")) return rc;
            hipLaunchKernelGGL(add_from_channels_last_kernel<T>, tgrid, tblock, 0, s, (const T*)gin_cl, gin, P.C_in, P.inV,
                               (const unsigned*)sel, (unsigned)MAX_PLANS);
            if (int rc = check_launch("add_from_channels_last_kernel")) return rc;
        }
        return DCN_OK;
    }
    if constexpr (S16) {
        if (declined) *declined = true;
        return DCN_OK;
    } else {

    // 2) grad_offset from the channels-last kernel, grad_input from the LDS-privatised scatter
    if (int rc = relayout<T>(P, w, wt, 1, s)) return rc;
    {   // zero tap slabs behind the last group
        const size_t used = (size_t)P.G * P.kV * P.Mp * P.Cgp, pad = (size_t)TAP_PAD * P.Mp * P.Cgp;
        hipLaunchKernelGGL(fill_zero_kernel<T>, dim3((unsigned)((pad + 255) / 256)), dim3(256), 0, s, wt + used, pad);
        if (int rc = check_launch("fill_zero_kernel")) return rc;
    }
    if (!input_only) {
        hipLaunchKernelGGL(to_channels_last_kernel<T>, tgrid, tblock, 0, s, in, in_cl, P.C_in, P.inV);
        if (int rc = check_launch("to_channels_last_kernel")) return rc;
    }
    Params Ph = P;
    bool halo = scatter_in_lds() && plan_halo<T, ND>(Ph, scatter_budget(), default_margin(), 8, 8);
    if (halo && (long long)Ph.N * Ph.tiles * Ph.DG > 0x7fffffffLL) halo = false;
    if (halo) {                                     // the scatter kernel packs 4 or 8 channels per MFMA tile
        const size_t fit = (scatter_budget() - (size_t)Ph.hvol * 4) / ((size_t)Ph.hstride * 8);
        if (fit >= 8) Ph.cchunk = 8;
        else if (fit >= 4) Ph.cchunk = 4;
        else halo = false;
    }
    P.tiles = (P.outV + WAVES * TN - 1) / (WAVES * TN);
    if ((long long)P.N * P.tiles > 0x7fffffffLL || P.DG > 65535)
        return fail(DCN_E_ARGUMENT, "layer too large for the kernel without the fused LDS halo (more than 65535 deformable groups)");
    const dim3 grid((unsigned)P.N * P.tiles, (unsigned)P.DG);
    if (halo) {
        T* none = nullptr;
        if (!input_only)
        switch (mk) {      // register-resident grad_output slab when M is small enough
            case 8: hipLaunchKernelGGL((backward_data_kernel<T, ND, false, 8>), grid, dim3(WG), 0, s, P, in_cl, off, wt, gout, none, goff); break;
            case 16: hipLaunchKernelGGL((backward_data_kernel<T, ND, false, 16>), grid, dim3(WG), 0, s, P, in_cl, off, wt, gout, none, goff); break;
            case 32: hipLaunchKernelGGL((backward_data_kernel<T, ND, false, 32>), grid, dim3(WG), 0, s, P, in_cl, off, wt, gout, none, goff); break;
            default: hipLaunchKernelGGL((backward_data_kernel<T, ND, false, 0>), grid, dim3(WG), 0, s, P, in_cl, off, wt, gout, none, goff); break;
        }
        if (!input_only)
            if (int rc = check_launch("backward_data_kernel")) return rc;
        const size_t lds = (size_t)Ph.cchunk * Ph.hstride * 8 + (size_t)Ph.hvol * 4;
        if (int rc = absmax<T>(w, (size_t)P.C_out * P.Cg * P.kV, wmax, s)) return rc;
        const dim3 hgrid((unsigned)Ph.N * Ph.tiles * Ph.DG);
        T* nogoff = nullptr;
        PlanSet alts;
        for (int e = 1; e < MAX_PLANS; ++e) alts.alt[e - 1] = halo_plan_of(Ph);
        alts.mask = 1u;
        const unsigned* nosel = nullptr;
        if (Ph.cchunk == 8)
            return launch_halo(backward_input_halo_kernel<T, ND, 8, false, false, 0, WAVESH>, "backward_input_halo_kernel", hgrid, WGH, lds, s,
                               Ph, alts, nosel, in, off, (const T*)wt, gout, (const float*)wmax, gin, nogoff, 1, 0u, 0);
        if (Ph.cchunk == 4)
            return launch_halo(backward_input_halo_kernel<T, ND, 4, false, false, 0, WAVESH>, "backward_input_halo_kernel", hgrid, WGH, lds, s,
                               Ph, alts, nosel, in, off, (const T*)wt, gout, (const float*)wmax, gin, nogoff, 1, 0u, 0);
        return fail(DCN_E_LAUNCH, "no scatter kernel for this channel chunk");
    }
    // halo does not fit in LDS: scatter with global atomics on the channels-last copy
    const size_t nelem = (size_t)P.N * P.C_in * P.inV;
    const unsigned fblocks = (unsigned)((nelem + 1023) / 1024 > 8192 ? 8192 : (nelem + 1023) / 1024);
    hipLaunchKernelGGL(fill_zero_kernel<T>, dim3(fblocks), dim3(256), 0, s, gin_cl, nelem);
    if (int rc = check_launch("fill_zero_kernel")) return rc;
    if (input_only) {       // the kernel reads input values for the grad_offset it also writes (into scratch here)
        hipLaunchKernelGGL(fill_zero_kernel<T>, dim3(fblocks), dim3(256), 0, s, in_cl, nelem);
        if (int rc = check_launch("fill_zero_kernel")) return rc;
    }
    hipLaunchKernelGGL((backward_data_kernel<T, ND, true, 0>), grid, dim3(WG), 0, s, P, in_cl, off, wt, gout, gin_cl, goff);
    if (int rc = check_launch("backward_data_kernel")) return rc;
    hipLaunchKernelGGL(add_from_channels_last_kernel<T>, tgrid, tblock, 0, s, gin_cl, gin, P.C_in, P.inV);
    return check_launch("add_from_channels_last_kernel");
    }
}

// Plan of backward_weight: channel tiles, m chunks and the number of position splits.
template <typename T>
void bww_plan(const Params& Pin, int& MT, int& mchunks, int& nct, int& nsplit, long long resident = 0) {
    const int TN = Mma<T>::TN;
    const int mtiles = (Pin.M + TN - 1) / TN;
    MT = mtiles > 2 ? 4 : mtiles;
    mchunks = (mtiles + MT - 1) / MT;
    // channel tiles: one per TN channels of every (convolution group x deformable group) segment
    nct = 0;
    for (int gg = 0; gg < Pin.G; ++gg) {
        const int cg0 = gg * Pin.Cg, cg1 = cg0 + Pin.Cg;
        for (int dg = cg0 / Pin.cpg; dg <= (cg1 - 1) / Pin.cpg; ++dg) {
            const int cb = cg0 > dg * Pin.cpg ? cg0 : dg * Pin.cpg;
            const int ce = cg1 < (dg + 1) * Pin.cpg ? cg1 : (dg + 1) * Pin.cpg;
            nct += (ce - cb + TN - 1) / TN;
        }
    }
    // split the position reduction so that the grid holds a few thousand workgroups: the largest
    // whole number of rounds of resident workgroups below about 2560 (a grid just past a whole
    // number of rounds pays a full round for the remainder; more splits mean more partial tiles to
    // write and add up: 4096 measured 1 to 7 % slower on the five benchmark layers)
    constexpr long long BWW_TARGET = 2560;
    const long long slabs = (long long)Pin.N * ((Pin.outV + TN - 1) / TN);
    const long long other = (long long)Pin.kV * nct * mchunks;
    long long split = (BWW_TARGET + other - 1) / other;
    if (resident > 0 && resident <= BWW_TARGET) {
        const long long balanced = (BWW_TARGET / resident) * resident / other;
        if (balanced >= 1 && balanced < split) split = balanced;
    }
    const long long max_split = (slabs + WAVES - 1) / WAVES;
    if (split > max_split) split = max_split;
    if (split > 256) split = 256;
    if (split < 1) split = 1;
    nsplit = (int)split;
}

// Workgroups of backward_weight_kernel that the device holds at once (0 if the query fails).
template <typename T, int ND, int MT>
long long bww_resident() {
    static const long long v = [] {
        int per_cu = 0;
        const size_t lds = (size_t)WAVES * Mma<T>::TN * (Mma<T>::TN + 1) * sizeof(T);
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, backward_weight_kernel<T, ND, MT>, WG, lds) != hipSuccess) {
            (void)hipGetLastError();
            return 0LL;
        }
        return (long long)per_cu * cu_count();
    }();
    return v;
}

template <typename T, int ND, int MT>
int launch_bwd_weight(const Params& P, const T* in_cl, const T* off, const T* gout_cl, T* partial, hipStream_t s) {
    const int TN = Mma<T>::TN;
    const size_t lds = (size_t)WAVES * TN * (TN + 1) * sizeof(T);
    auto kern = backward_weight_kernel<T, ND, MT>;
    if (lds > 48 * 1024)
        if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kern), lds)) return rc;
    const dim3 grid((unsigned)P.nsplit * P.kV * P.nctiles * P.mchunks);
    hipLaunchKernelGGL(kern, grid, dim3(WG), lds, s, P, in_cl, off, gout_cl, partial);
    return check_launch("backward_weight_kernel");
}

template <typename T> size_t bww_workspace(const Params& P, int nsplit) {
    return align256((size_t)P.N * P.C_in * P.inV * sizeof(T)) + align256((size_t)P.N * P.C_out * P.outV * sizeof(T)) +
           align256((size_t)nsplit * P.kV * P.C_out * P.Cg * sizeof(T));
}

// Workspace of backward_weight: [ input channels-last | grad_output channels-last | partial tiles per split ]
template <typename T, int ND>
int backward_weight(const Geometry& g, const T* in, const T* off, const T* gout, T* gw, void* ws, size_t ws_bytes,
                    hipStream_t s) {
    Params P;
    if (int rc = validate(g, P)) return rc;
    if (!in || !off || !gout || !gw) return fail(DCN_E_ARGUMENT, "null tensor pointer");
    if (int rc = device_info(nullptr)) return rc;
    if ((long long)P.outV * P.C_out > (1ll << 31)) return fail(DCN_E_ARGUMENT, "one output sample exceeds 2^31 elements");
    // (the layout change of both operands is one launch with 2 * N slices along z)
    if (2 * (long long)P.N > 65535) return fail(DCN_E_ARGUMENT, "backward_weight: batch exceeds 32767");
    // the kernel addresses both operands by 32-bit byte offsets from the sample's base
    if ((unsigned long long)P.inV * P.C_in * sizeof(T) >= (1ull << 32) || (unsigned long long)P.outV * P.C_out * sizeof(T) >= (1ull << 32))
        return fail(DCN_E_ARGUMENT, "one sample of the input or of grad_output reaches 4 GiB");
    int MT;
    bww_plan<T>(P, MT, P.mchunks, P.nctiles, P.nsplit);
    const long long resident = MT == 1 ? bww_resident<T, ND, 1>() : MT == 2 ? bww_resident<T, ND, 2>() : bww_resident<T, ND, 4>();
    bww_plan<T>(P, MT, P.mchunks, P.nctiles, P.nsplit, resident);
    if ((long long)P.nsplit * P.kV * P.nctiles * P.mchunks > 0x7fffffffLL) return fail(DCN_E_ARGUMENT, "too many workgroups for one launch");
    const size_t ibytes = align256((size_t)P.N * P.C_in * P.inV * sizeof(T));
    const size_t obytes = align256((size_t)P.N * P.C_out * P.outV * sizeof(T));
    if (!ws || ws_bytes < bww_workspace<T>(P, P.nsplit)) return fail(DCN_E_WORKSPACE, "workspace too small");
    T* in_cl = static_cast<T*>(ws);
    T* gout_cl = reinterpret_cast<T*>(static_cast<char*>(ws) + ibytes);
    T* partial = reinterpret_cast<T*>(static_cast<char*>(ws) + ibytes + obytes);
    const dim3 tblock(32, 8);
    {
        const unsigned vmax = P.inV > P.outV ? P.inV : P.outV;
        const int cmax = P.C_in > P.C_out ? P.C_in : P.C_out;
        hipLaunchKernelGGL(to_channels_last_pair_kernel<T>, dim3((vmax + 31) / 32, (unsigned)(cmax + 31) / 32, 2u * (unsigned)P.N), tblock, 0, s,
                           in, in_cl, P.C_in, P.inV, gout, gout_cl, P.C_out, P.outV, P.N);
        if (int rc = check_launch("to_channels_last_pair_kernel")) return rc;
    }
    int rc;
    switch (MT) {
        case 1: rc = launch_bwd_weight<T, ND, 1>(P, in_cl, off, gout_cl, partial, s); break;
        case 2: rc = launch_bwd_weight<T, ND, 2>(P, in_cl, off, gout_cl, partial, s); break;
        default: rc = launch_bwd_weight<T, ND, 4>(P, in_cl, off, gout_cl, partial, s); break;
    }
    if (rc) return rc;
    const size_t rows_x_cg = (size_t)P.C_out * P.Cg, total = rows_x_cg * P.kV;
    const unsigned rb = (unsigned)((total + 63) / 64 > 8192 ? 8192 : (total + 63) / 64);
    hipLaunchKernelGGL(reduce_weight_partials_kernel<T>, dim3(rb), dim3(256), 0, s, partial, gw, P.nsplit, P.kV, rows_x_cg);
    return check_launch("reduce_weight_partials_kernel");
}

// ---------------------------------------------------------------------------------------------
// Mixed precision: tensors stored as bfloat16 / binary16, accumulation in float32.  Each call first
// offers the layer to the kernel that reads the 16-bit tensors itself and multiplies on the 16-bit
// matrix instructions (float results in a float copy at the front of the workspace, rounded once
// when they are written back); where that kernel declines, the tensors are widened into float
// copies at the front of the workspace and the float32 kernels run on them with the rest of it.
struct Carver {
    char* p;
    size_t left;
    float* take(size_t n) {
        const size_t b = align256(n * sizeof(float));
        if (!p || b > left) return nullptr;
        float* r = reinterpret_cast<float*>(p);
        p += b;
        left -= b;
        return r;
    }
};
template <typename S> int widen(const S* src, float* dst, size_t n, hipStream_t s) {
    const unsigned blocks = (unsigned)((n + 1023) / 1024 > 8192 ? 8192 : (n + 1023) / 1024);
    hipLaunchKernelGGL(widen_kernel<S>, dim3(blocks ? blocks : 1), dim3(256), 0, s, src, dst, n);
    return check_launch("widen_kernel");
}
template <typename S> int narrow(const float* src, S* dst, size_t n, hipStream_t s) {
    const unsigned blocks = (unsigned)((n + 1023) / 1024 > 8192 ? 8192 : (n + 1023) / 1024);
    hipLaunchKernelGGL(narrow_kernel<S>, dim3(blocks ? blocks : 1), dim3(256), 0, s, src, dst, n);
    return check_launch("narrow_kernel");
}
struct Sizes16 { size_t in, w, off, out; };
Sizes16 sizes16(const Params& P, int nd) {
    return Sizes16{(size_t)P.N * P.C_in * P.inV, (size_t)P.C_out * P.Cg * P.kV, (size_t)P.N * P.DG * P.kV * nd * P.outV,
                   (size_t)P.N * P.C_out * P.outV};
}
// float copies of every tensor any of the three calls touches (nd = 3 bounds the offsets of either operator)
size_t copies16_bytes(int N, int C_in, int C_out, size_t inV, size_t outV, int kV, int G, int cpg) {
    const size_t in = (size_t)N * C_in * inV, w = (size_t)C_out * (C_in / G) * kV, off = (size_t)N * (C_in / cpg) * kV * 3 * outV,
                 out = (size_t)N * C_out * outV;
    return 2 * align256(in * 4) + 2 * align256(w * 4) + 2 * align256(off * 4) + align256(out * 4) + align256((size_t)C_out * 4);
}

template <typename S, int ND>
int forward16(const Geometry& g, const S* in, const S* w, const S* off, const S* bias, S* out, void* ws, size_t ws_bytes,
              hipStream_t s) {
    Params P;
    if (int rc = validate(g, P)) return rc;
    if (!in || !w || !off || !out) return fail(DCN_E_ARGUMENT, "null tensor pointer");
    if (int rc = device_info(nullptr)) return rc;
    if (native16()) {       // the LDS-halo kernel reads the 16-bit tensors itself and multiplies with 16-bit matrix instructions
        bool declined = false;
        if (int rc = forward<float, ND, S>(g, in, w, off, bias, out, ws, ws_bytes, s, &declined)) return rc;
        if (!declined) return DCN_OK;
    }
    const Sizes16 z = sizes16(P, ND);
    Carver c{static_cast<char*>(ws), ws ? ws_bytes : 0};
    float *fin = c.take(z.in), *fw = c.take(z.w), *foff = c.take(z.off), *fout = c.take(z.out), *fb = bias ? c.take(P.C_out) : nullptr;
    if (!fin || !fw || !foff || !fout || (bias && !fb)) return fail(DCN_E_WORKSPACE, "workspace too small");
    if (int rc = widen(in, fin, z.in, s)) return rc;
    if (int rc = widen(w, fw, z.w, s)) return rc;
    if (int rc = widen(off, foff, z.off, s)) return rc;
    if (bias) if (int rc = widen(bias, fb, (size_t)P.C_out, s)) return rc;
    if (int rc = forward<float, ND>(g, fin, fw, foff, fb, fout, c.p, c.left, s)) return rc;
    return narrow(fout, out, z.out, s);
}
template <typename S, int ND>
int backward_input_offset16(const Geometry& g, const S* in, const S* w, const S* off, const S* gout, S* gin, S* goff, void* ws,
                            size_t ws_bytes, hipStream_t s) {
    Params P;
    if (int rc = validate(g, P)) return rc;
    if (!in || !w || !off || !gout || !gin || !goff) return fail(DCN_E_ARGUMENT, "null tensor pointer");
    if (int rc = device_info(nullptr)) return rc;
    const Sizes16 z = sizes16(P, ND);
    Carver c{static_cast<char*>(ws), ws ? ws_bytes : 0};
    float *fin = c.take(z.in), *fw = c.take(z.w), *foff = c.take(z.off), *fgout = c.take(z.out), *fgin = c.take(z.in), *fgoff = c.take(z.off);
    if (!fin || !fw || !foff || !fgout || !fgin || !fgoff) return fail(DCN_E_WORKSPACE, "workspace too small");
    if (int rc = widen(gin, fgin, z.in, s)) return rc;            // grad_input is accumulated into
    // the fused kernel reads the 16-bit tensors itself and forms the grad columns with 16-bit matrix
    // instructions (the products of 16-bit values are exact in float, so the results are those of the
    // float32 kernel up to the order of the sums); the gradients leave it as float and are rounded once
    bool declined = true;
    if (native16()) {
        declined = false;
        if (int rc = backward_input_offset<float, ND, S>(g, in, w, off, gout, fgin, fgoff, c.p, c.left, s, 0, &declined)) return rc;
    }
    if (declined) {
        if (int rc = widen(in, fin, z.in, s)) return rc;
        if (int rc = widen(w, fw, z.w, s)) return rc;
        if (int rc = widen(off, foff, z.off, s)) return rc;
        if (int rc = widen(gout, fgout, z.out, s)) return rc;
        if (int rc = backward_input_offset<float, ND>(g, fin, fw, foff, fgout, fgin, fgoff, c.p, c.left, s)) return rc;
    }
    if (int rc = narrow(fgin, gin, z.in, s)) return rc;
    return narrow(fgoff, goff, z.off, s);
}
// backward_weight on the 16-bit tensors themselves (backward_weight16_kernel): channels-last copies of
// the input and of grad_output in their storage format, the offsets as they are, float partial tiles.
// Declines (nothing launched) where the kernel's 4-byte loads of channel pairs would not be aligned
// (an odd number of input channels, or segments -- intersections of convolution groups and deformable
// groups -- that start at odd channels) or the workspace is too small for it.
template <typename S, int ND>
int backward_weight_native16(const Params& Pin, const S* in, const S* off, const S* gout, float* fgw, void* ws, size_t ws_bytes,
                             hipStream_t s, bool* declined) {
    Params P = Pin;
    const int TN = Mma<float>::TN, CT = 2 * TN;
    *declined = true;
    if (P.C_in % 2 || P.cpg % 2 || P.Cg % 2) return DCN_OK;
    if ((unsigned long long)P.inV * P.C_in * sizeof(S) >= (1ull << 32) || (unsigned long long)P.outV * P.C_out >= (1ull << 32)) return DCN_OK;
    if (2 * (long long)P.N > 65535) return DCN_OK;
    const int mtiles = (P.M + TN - 1) / TN;
    // Two row tiles per workgroup at most (four would take 128 accumulator registers beside the two
    // channel tiles: one wavefront per SIMD), so more than 64 output channels sample everything once
    // per 64 of them, and channel segments that fill their 64-channel tiles badly waste the lanes'
    // loads.  Both kernels are bounded by their corner loads: this one issues half as many per
    // channel as the float32 kernel (four row tiles, 32-channel tiles), times the re-sampling and the
    // unused part of the tiles.  Where that comes to more than the float32 kernel's, that kernel on
    // widened tensors is the faster one (128 -> 128 channels in deformable groups of 32, 3-D: 2.5 ms
    // here against 1.2 + 0.15 for widening; 256 -> 256 in one group, 2-D: 0.20 here against 0.31).
    const int MT = mtiles >= 2 ? 2 : 1;
    P.mchunks = (mtiles + MT - 1) / MT;
    P.nctiles = 0;
    int nct32 = 0;
    for (int gg = 0; gg < P.G; ++gg) {
        const int cg0 = gg * P.Cg, cg1 = cg0 + P.Cg;
        for (int dg = cg0 / P.cpg; dg <= (cg1 - 1) / P.cpg; ++dg) {
            const int cb = cg0 > dg * P.cpg ? cg0 : dg * P.cpg, ce = cg1 < (dg + 1) * P.cpg ? cg1 : (dg + 1) * P.cpg;
            P.nctiles += (ce - cb + CT - 1) / CT;
            nct32 += (ce - cb + TN - 1) / TN;
        }
    }
    {
        const long long loads16 = (long long)P.mchunks * P.nctiles, loads32 = (long long)((mtiles + 3) / 4) * nct32;
        if (4 * loads16 > 5 * loads32) return DCN_OK;
    }
    // position splits: about 2560 workgroups, as in the float kernel's plan
    const long long slabs = (long long)P.N * ((P.outV + TN - 1) / TN), other = (long long)P.kV * P.nctiles * P.mchunks;
    long long split = (2560 + other - 1) / other;
    const long long max_split = (slabs + WAVES - 1) / WAVES;
    if (split > max_split) split = max_split;
    if (split > 256) split = 256;
    if (split < 1) split = 1;
    P.nsplit = (int)split;
    if ((long long)P.nsplit * other > 0x7fffffffLL) return DCN_OK;
    const size_t ibytes = align256((size_t)P.N * P.C_in * P.inV * sizeof(S));
    const size_t obytes = align256((size_t)P.N * P.C_out * P.outV * sizeof(S));
    const size_t pbytes = align256((size_t)P.nsplit * P.kV * P.C_out * P.Cg * sizeof(float));
    if (!ws || ws_bytes < ibytes + obytes + pbytes) return DCN_OK;
    *declined = false;
    S* in_cl = static_cast<S*>(ws);
    S* gout_cl = reinterpret_cast<S*>(static_cast<char*>(ws) + ibytes);
    float* partial = reinterpret_cast<float*>(static_cast<char*>(ws) + ibytes + obytes);
    {
        const unsigned vmax = P.inV > P.outV ? P.inV : P.outV;
        const int cmax = P.C_in > P.C_out ? P.C_in : P.C_out;
        hipLaunchKernelGGL(to_channels_last_pair_kernel<S>, dim3((vmax + 31) / 32, (unsigned)(cmax + 31) / 32, 2u * (unsigned)P.N), dim3(32, 8), 0, s,
                           in, in_cl, P.C_in, P.inV, gout, gout_cl, P.C_out, P.outV, P.N);
        if (int rc = check_launch("to_channels_last_pair_kernel")) return rc;
    }
    const size_t lds = (size_t)WAVES * TN * (TN + 1) * sizeof(float);
    const dim3 grid((unsigned)(P.nsplit * other));
    if (MT == 2) hipLaunchKernelGGL((backward_weight16_kernel<ND, 2, S>), grid, dim3(WG), lds, s, P, (const S*)in_cl, off, (const S*)gout_cl, partial);
    else hipLaunchKernelGGL((backward_weight16_kernel<ND, 1, S>), grid, dim3(WG), lds, s, P, (const S*)in_cl, off, (const S*)gout_cl, partial);
    if (int rc = check_launch("backward_weight16_kernel")) return rc;
    const size_t rows_x_cg = (size_t)P.C_out * P.Cg, total = rows_x_cg * P.kV;
    const unsigned rb = (unsigned)((total + 63) / 64 > 8192 ? 8192 : (total + 63) / 64);
    hipLaunchKernelGGL(reduce_weight_partials_kernel<float>, dim3(rb), dim3(256), 0, s, (const float*)partial, fgw, P.nsplit, P.kV, rows_x_cg);
    return check_launch("reduce_weight_partials_kernel");
}

template <typename S, int ND>
int backward_weight16(const Geometry& g, const S* in, const S* off, const S* gout, S* gw, void* ws, size_t ws_bytes, hipStream_t s) {
    Params P;
    if (int rc = validate(g, P)) return rc;
    if (!in || !off || !gout || !gw) return fail(DCN_E_ARGUMENT, "null tensor pointer");
    if (int rc = device_info(nullptr)) return rc;
    const Sizes16 z = sizes16(P, ND);
    Carver c{static_cast<char*>(ws), ws ? ws_bytes : 0};
    float *fin = c.take(z.in), *foff = c.take(z.off), *fgout = c.take(z.out), *fgw = c.take(z.w);
    if (!fin || !foff || !fgout || !fgw) return fail(DCN_E_WORKSPACE, "workspace too small");
    if (int rc = widen(gw, fgw, z.w, s)) return rc;               // grad_weight is accumulated into
    bool declined = true;
    if (native16())
        if (int rc = backward_weight_native16<S, ND>(P, in, off, gout, fgw, c.p, c.left, s, &declined)) return rc;
    if (declined) {
        if (int rc = widen(in, fin, z.in, s)) return rc;
        if (int rc = widen(off, foff, z.off, s)) return rc;
        if (int rc = widen(gout, fgout, z.out, s)) return rc;
        if (int rc = backward_weight<float, ND>(g, fin, foff, fgout, fgw, c.p, c.left, s)) return rc;
    }
    return narrow(fgw, gw, z.w, s);
}

// ---------------------------------------------------------------------------------------------
// Plain 2-D convolution: the reference's conv2d package (conv2d/lib/conv2d_cuda.cpp:77-290, kernels
// conv2d/lib/conv2d_cuda_kernel.cu:25-169: im2col / col2im with integer taps and one GEMM per sample
// and group).  It is the 2-D deformable layer with every offset zero, one deformable group and the
// dilation-aware output size (conv2d/lib/conv2d_cuda.cpp:20-22), so it runs on the same kernels: a
// zero offset tensor at the front of the workspace, behind it scratch for the grad_offset that
// one fallback kernel of backward-to-input writes, then the deformable layer's own workspace.
template <typename T> size_t conv2d_zero_bytes(int N, int kV, size_t outV) { return align256((size_t)N * 2 * kV * outV * sizeof(T)); }
template <typename T>
int conv2d_offsets(const Geometry& g, void* ws, size_t ws_bytes, hipStream_t s, T** off, T** scratch, void** rest, size_t* rest_bytes) {
    if (g.N <= 0 || g.out[1] <= 0 || g.out[2] <= 0 || g.k[1] <= 0 || g.k[2] <= 0) return fail(DCN_E_ARGUMENT, "batch / output / kernel extents must be positive");
    const size_t zb = conv2d_zero_bytes<T>(g.N, g.k[1] * g.k[2], (size_t)g.out[1] * g.out[2]);
    if (!ws || ws_bytes < 2 * zb) return fail(DCN_E_WORKSPACE, "workspace too small");
    *off = static_cast<T*>(ws);
    *scratch = reinterpret_cast<T*>(static_cast<char*>(ws) + zb);
    *rest = static_cast<char*>(ws) + 2 * zb;
    *rest_bytes = ws_bytes - 2 * zb;
    const size_t n = zb / sizeof(T);
    const unsigned blocks = (unsigned)((n + 1023) / 1024 > 4096 ? 4096 : (n + 1023) / 1024);
    hipLaunchKernelGGL(fill_zero_kernel<T>, dim3(blocks), dim3(256), 0, s, *off, n);
    return check_launch("fill_zero_kernel");
}
template <typename T>
int conv2d_forward(Geometry g, const T* in, const T* w, const T* bias, T* out, void* ws, size_t ws_bytes, hipStream_t s) {
    g.cpg = g.C_in;
    T *off, *scratch; void* rest; size_t rest_bytes;
    if (int rc = conv2d_offsets<T>(g, ws, ws_bytes, s, &off, &scratch, &rest, &rest_bytes)) return rc;
    return forward<T, 2>(g, in, w, off, bias, out, rest, rest_bytes, s);
}
template <typename T>
int conv2d_backward_input(Geometry g, const T* w, const T* gout, T* gin, void* ws, size_t ws_bytes, hipStream_t s) {
    g.cpg = g.C_in;
    T *off, *scratch; void* rest; size_t rest_bytes;
    if (int rc = conv2d_offsets<T>(g, ws, ws_bytes, s, &off, &scratch, &rest, &rest_bytes)) return rc;
    return backward_input_offset<T, 2>(g, static_cast<const T*>(nullptr), w, static_cast<const T*>(off), gout, gin, scratch, rest, rest_bytes, s, FLAG_INPUT_ONLY);
}
template <typename T>
int conv2d_backward_weight(Geometry g, const T* in, const T* gout, T* gw, void* ws, size_t ws_bytes, hipStream_t s) {
    g.cpg = g.C_in;
    T *off, *scratch; void* rest; size_t rest_bytes;
    if (int rc = conv2d_offsets<T>(g, ws, ws_bytes, s, &off, &scratch, &rest, &rest_bytes)) return rc;
    return backward_weight<T, 2>(g, in, off, gout, gw, rest, rest_bytes, s);
}

Geometry geo3(int batch, int input_c, int output_c, int input_l, int input_h, int input_w, int output_l,
              int output_h, int output_w, int kernel_l, int kernel_h, int kernel_w, int pad_l, int pad_h,
              int pad_w, int stride_l, int stride_h, int stride_w, int dilation_l, int dilation_h,
              int dilation_w, int cpg, int group) {
    return Geometry{3, batch, input_c, output_c, {input_l, input_h, input_w}, {output_l, output_h, output_w},
                    {kernel_l, kernel_h, kernel_w}, {pad_l, pad_h, pad_w}, {stride_l, stride_h, stride_w},
                    {dilation_l, dilation_h, dilation_w}, cpg, group};
}
Geometry geo2(int batch, int input_c, int output_c, int input_h, int input_w, int output_h, int output_w,
              int kernel_h, int kernel_w, int pad_h, int pad_w, int stride_h, int stride_w, int dilation_h,
              int dilation_w, int cpg, int group) {
    return Geometry{2, batch, input_c, output_c, {1, input_h, input_w}, {1, output_h, output_w},
                    {1, kernel_h, kernel_w}, {0, pad_h, pad_w}, {1, stride_h, stride_w},
                    {1, dilation_h, dilation_w}, cpg, group};
}

// ---------------------------------------------------------------------------------------------
// Scratch of the allocation-free entry point: the re-laid-out weight of one forward call.  A
// file-scope device array, so every GPU the library runs on holds DCN_NOALLOC_SCRATCH_BYTES of it
// until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress: the device address is looked up once per device and kept, and host code
// passes that address, never the name, to kernels.
static __device__ __align__(256) unsigned char scratch[DCN_NOALLOC_SCRATCH_BYTES];

std::mutex g_scratch_lock;
void* g_scratch_ptr[MAX_DEVICES] = {};

int scratch_address(void** out) {
    int dev = -1;
    if (int rc = device_info(nullptr, &dev)) return rc;
    std::lock_guard<std::mutex> lock(g_scratch_lock);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            (void)hipGetLastError();
            g_err = std::string("hipGetSymbolAddress(scratch): ") + hipGetErrorString(e);
            return DCN_E_DEVICE;
        }
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return DCN_OK;
}

}  // namespace

#define G3_ARGS batch, input_c, output_c, input_l, input_h, input_w, output_l, output_h, output_w, kernel_l, \
                kernel_h, kernel_w, pad_l, pad_h, pad_w, stride_l, stride_h, stride_w, dilation_l, dilation_h, \
                dilation_w, channel_per_deformable_group, group
#define G2_ARGS batch, input_c, output_c, input_h, input_w, output_h, output_w, kernel_h, kernel_w, pad_h, pad_w, \
                stride_h, stride_w, dilation_h, dilation_w, channel_per_deformable_group, group

extern "C" {

int dcn_version(void) { return 1; }
const char* dcn_arch(void) { return "gfx950"; }
const char* dcn_last_error(void) { return g_err.c_str(); }

size_t dcn_workspace_bytes(int elem_size, int batch, int input_c, int output_c, size_t input_volume,
                           size_t output_volume, int kernel_volume, int group) {
    if (group <= 0 || batch <= 0 || input_c <= 0 || output_c <= 0 || kernel_volume <= 0 || input_volume == 0 ||
        output_volume == 0 || elem_size == 2)      // 16-bit storage: dcn_workspace_bytes_for
        return 0;
    return elem_size == 8
               ? workspace_need<double>(batch, input_c, output_c, input_volume, output_volume, kernel_volume, group)
               : workspace_need<float>(batch, input_c, output_c, input_volume, output_volume, kernel_volume, group);
}

size_t dcn_workspace_bytes_for(int elem_size, int batch, int input_c, int output_c, size_t input_volume,
                               size_t output_volume, int kernel_volume, int group, int channel_per_deformable_group) {
    if (group <= 0 || batch <= 0 || input_c <= 0 || output_c <= 0 || kernel_volume <= 0 || input_volume == 0 ||
        output_volume == 0 || channel_per_deformable_group <= 0 || input_c % channel_per_deformable_group)
        return 0;
    const int cpg = channel_per_deformable_group;
    if (elem_size == 2)     // bfloat16 / binary16 storage: float copies of the tensors + the float32 workspace
        return copies16_bytes(batch, input_c, output_c, input_volume, output_volume, kernel_volume, group, cpg) +
               workspace_need<float>(batch, input_c, output_c, input_volume, output_volume, kernel_volume, group, cpg);
    return elem_size == 8
               ? workspace_need<double>(batch, input_c, output_c, input_volume, output_volume, kernel_volume, group, cpg)
               : workspace_need<float>(batch, input_c, output_c, input_volume, output_volume, kernel_volume, group, cpg);
}

int dcn3d_forward_noalloc_f32(const float* input, const float* weight, const float* offset, const float* bias,
                              float* output, DCN3D_GEOMETRY, void* stream) {
    const Geometry g = geo3(G3_ARGS);
    Params P;
    if (int rc = validate(g, P)) return rc;
    // what forward() asks of a workspace: either weight layout must fit the fixed array
    int MT, mchunks, Mp, Cgp;
    fwd_weight_pad<float>(P.M, P.Cg, MT, mchunks, Mp, Cgp);
    const int Mp8 = ((P.M + 31) / 32 + 7) / 8 * 8 * 32;
    const size_t plain = (size_t)P.G * P.kV * (Mp > Mp8 ? Mp : Mp8) * Cgp * sizeof(float);
    const size_t quad = ((size_t)chunk_slot<FQ>(P.cpg, P.Cg, P.C_in - 1) + 1) * forward_slab_elems<float>(P.kV, Mp8) * sizeof(float);
    if (plain > DCN_NOALLOC_SCRATCH_BYTES || quad > DCN_NOALLOC_SCRATCH_BYTES) {
        char msg[200];
        snprintf(msg, sizeof msg, "layer too large for the allocation-free entry point: its re-laid-out weight takes %zu bytes, "
                 "the fixed scratch holds %zu", plain > quad ? plain : quad, (size_t)DCN_NOALLOC_SCRATCH_BYTES);
        return fail(DCN_E_WORKSPACE, msg);
    }
    void* ws = nullptr;
    if (int rc = scratch_address(&ws)) return rc;
    return forward<float, 3>(g, input, weight, offset, bias, output, ws, DCN_NOALLOC_SCRATCH_BYTES,
                             static_cast<hipStream_t>(stream));
}

#define DEFINE_OPS(SUF, T)                                                                                          \
    int dcn3d_forward_##SUF(const T* input, const T* weight, const T* offset, const T* bias, T* output,             \
                            DCN3D_GEOMETRY, void* workspace, size_t workspace_bytes, void* stream) {                \
        return forward<T, 3>(geo3(G3_ARGS), input, weight, offset, bias, output, workspace, workspace_bytes,        \
                             static_cast<hipStream_t>(stream));                                                     \
    }                                                                                                               \
    int dcn3d_backward_input_offset_##SUF(const T* input, const T* weight, const T* offset, const T* grad_output,   \
                                          T* grad_input, T* grad_offset, DCN3D_GEOMETRY, void* workspace,           \
                                          size_t workspace_bytes, void* stream) {                                   \
        return backward_input_offset<T, 3>(geo3(G3_ARGS), input, weight, offset, grad_output, grad_input,           \
                                           grad_offset, workspace, workspace_bytes,                                 \
                                           static_cast<hipStream_t>(stream));                                       \
    }                                                                                                               \
    int dcn3d_backward_input_offset_flags_##SUF(const T* input, const T* weight, const T* offset,                   \
                                                const T* grad_output, T* grad_input, T* grad_offset,                \
                                                DCN3D_GEOMETRY, void* workspace, size_t workspace_bytes,            \
                                                void* stream, unsigned flags) {                                     \
        if (flags & ~(unsigned)DCN_FLAG_OOB_OFFSET_GRAD_ZERO) return fail(DCN_E_ARGUMENT, "unknown flag");          \
        return backward_input_offset<T, 3>(geo3(G3_ARGS), input, weight, offset, grad_output, grad_input,           \
                                           grad_offset, workspace, workspace_bytes,                                 \
                                           static_cast<hipStream_t>(stream), flags);                                \
    }                                                                                                               \
    int dcn3d_backward_weight_##SUF(const T* input, const T* offset, const T* grad_output, T* grad_weight,          \
                                    DCN3D_GEOMETRY, void* workspace, size_t workspace_bytes, void* stream) {        \
        return backward_weight<T, 3>(geo3(G3_ARGS), input, offset, grad_output, grad_weight, workspace,             \
                                     workspace_bytes, static_cast<hipStream_t>(stream));                            \
    }                                                                                                               \
    int dcn2d_forward_##SUF(const T* input, const T* weight, const T* offset, const T* bias, T* output,             \
                            DCN2D_GEOMETRY, void* workspace, size_t workspace_bytes, void* stream) {                \
        return forward<T, 2>(geo2(G2_ARGS), input, weight, offset, bias, output, workspace, workspace_bytes,        \
                             static_cast<hipStream_t>(stream));                                                     \
    }                                                                                                               \
    int dcn2d_backward_input_offset_##SUF(const T* input, const T* weight, const T* offset, const T* grad_output,   \
                                          T* grad_input, T* grad_offset, DCN2D_GEOMETRY, void* workspace,           \
                                          size_t workspace_bytes, void* stream) {                                   \
        return backward_input_offset<T, 2>(geo2(G2_ARGS), input, weight, offset, grad_output, grad_input,           \
                                           grad_offset, workspace, workspace_bytes,                                 \
                                           static_cast<hipStream_t>(stream));                                       \
    }                                                                                                               \
    int dcn2d_backward_weight_##SUF(const T* input, const T* offset, const T* grad_output, T* grad_weight,          \
                                    DCN2D_GEOMETRY, void* workspace, size_t workspace_bytes, void* stream) {        \
        return backward_weight<T, 2>(geo2(G2_ARGS), input, offset, grad_output, grad_weight, workspace,             \
                                     workspace_bytes, static_cast<hipStream_t>(stream));                            \
    }

DEFINE_OPS(f32, float)
DEFINE_OPS(f64, double)

size_t conv2d_workspace_bytes(int elem_size, int batch, int input_c, int output_c, size_t input_volume, size_t output_volume,
                              int kernel_volume, int group) {
    const size_t inner = dcn_workspace_bytes_for(elem_size, batch, input_c, output_c, input_volume, output_volume, kernel_volume,
                                                 group, input_c);
    if (!inner || elem_size == 2) return 0;
    const size_t zb = elem_size == 8 ? conv2d_zero_bytes<double>(batch, kernel_volume, output_volume)
                                     : conv2d_zero_bytes<float>(batch, kernel_volume, output_volume);
    return inner + 2 * zb;
}
#define C2_ARGS batch, input_c, output_c, input_h, input_w, output_h, output_w, kernel_h, kernel_w, pad_h, pad_w, \
                stride_h, stride_w, dilation_h, dilation_w, input_c, group
#define DEFINE_CONV2D(SUF, T)                                                                                       \
    int conv2d_forward_##SUF(const T* input, const T* weight, const T* bias, T* output, CONV2D_GEOMETRY,            \
                             void* workspace, size_t workspace_bytes, void* stream) {                               \
        return conv2d_forward<T>(geo2(C2_ARGS), input, weight, bias, output, workspace, workspace_bytes,            \
                                 static_cast<hipStream_t>(stream));                                                 \
    }                                                                                                               \
    int conv2d_backward_input_##SUF(const T* weight, const T* grad_output, T* grad_input, CONV2D_GEOMETRY,          \
                                    void* workspace, size_t workspace_bytes, void* stream) {                        \
        return conv2d_backward_input<T>(geo2(C2_ARGS), weight, grad_output, grad_input, workspace, workspace_bytes, \
                                        static_cast<hipStream_t>(stream));                                          \
    }                                                                                                               \
    int conv2d_backward_weight_##SUF(const T* input, const T* grad_output, T* grad_weight, CONV2D_GEOMETRY,         \
                                     void* workspace, size_t workspace_bytes, void* stream) {                       \
        return conv2d_backward_weight<T>(geo2(C2_ARGS), input, grad_output, grad_weight, workspace,                 \
                                         workspace_bytes, static_cast<hipStream_t>(stream));                        \
    }
DEFINE_CONV2D(f32, float)
DEFINE_CONV2D(f64, double)

#define DEFINE_OPS16(SUF, S)                                                                                        \
    int dcn3d_forward_##SUF(const void* input, const void* weight, const void* offset, const void* bias, void* output, \
                            DCN3D_GEOMETRY, void* workspace, size_t workspace_bytes, void* stream) {                \
        return forward16<S, 3>(geo3(G3_ARGS), (const S*)input, (const S*)weight, (const S*)offset, (const S*)bias,  \
                               (S*)output, workspace, workspace_bytes, static_cast<hipStream_t>(stream));           \
    }                                                                                                               \
    int dcn3d_backward_input_offset_##SUF(const void* input, const void* weight, const void* offset,                \
                                          const void* grad_output, void* grad_input, void* grad_offset,             \
                                          DCN3D_GEOMETRY, void* workspace, size_t workspace_bytes, void* stream) {  \
        return backward_input_offset16<S, 3>(geo3(G3_ARGS), (const S*)input, (const S*)weight, (const S*)offset,    \
                                             (const S*)grad_output, (S*)grad_input, (S*)grad_offset, workspace,     \
                                             workspace_bytes, static_cast<hipStream_t>(stream));                    \
    }                                                                                                               \
    int dcn3d_backward_weight_##SUF(const void* input, const void* offset, const void* grad_output,                 \
                                    void* grad_weight, DCN3D_GEOMETRY, void* workspace, size_t workspace_bytes,     \
                                    void* stream) {                                                                 \
        return backward_weight16<S, 3>(geo3(G3_ARGS), (const S*)input, (const S*)offset, (const S*)grad_output,     \
                                       (S*)grad_weight, workspace, workspace_bytes,                                 \
                                       static_cast<hipStream_t>(stream));                                           \
    }                                                                                                               \
    int dcn2d_forward_##SUF(const void* input, const void* weight, const void* offset, const void* bias, void* output, \
                            DCN2D_GEOMETRY, void* workspace, size_t workspace_bytes, void* stream) {                \
        return forward16<S, 2>(geo2(G2_ARGS), (const S*)input, (const S*)weight, (const S*)offset, (const S*)bias,  \
                               (S*)output, workspace, workspace_bytes, static_cast<hipStream_t>(stream));           \
    }                                                                                                               \
    int dcn2d_backward_input_offset_##SUF(const void* input, const void* weight, const void* offset,                \
                                          const void* grad_output, void* grad_input, void* grad_offset,             \
                                          DCN2D_GEOMETRY, void* workspace, size_t workspace_bytes, void* stream) {  \
        return backward_input_offset16<S, 2>(geo2(G2_ARGS), (const S*)input, (const S*)weight, (const S*)offset,    \
                                             (const S*)grad_output, (S*)grad_input, (S*)grad_offset, workspace,     \
                                             workspace_bytes, static_cast<hipStream_t>(stream));                    \
    }                                                                                                               \
    int dcn2d_backward_weight_##SUF(const void* input, const void* offset, const void* grad_output,                 \
                                    void* grad_weight, DCN2D_GEOMETRY, void* workspace, size_t workspace_bytes,     \
                                    void* stream) {                                                                 \
        return backward_weight16<S, 2>(geo2(G2_ARGS), (const S*)input, (const S*)offset, (const S*)grad_output,     \
                                       (S*)grad_weight, workspace, workspace_bytes,                                 \
                                       static_cast<hipStream_t>(stream));                                           \
    }

DEFINE_OPS16(bf16, Bf16)
DEFINE_OPS16(f16, Fp16)

}  // extern "C"
