// Issue-rate probe for the vector ALU: what one SIMD sustains for the instructions the scan kernels are
// made of. Each wave runs `iters` rounds of 64 independent instructions of one kind on eight registers;
// the workgroups (four waves, one per SIMD) are sized so that `waves_per_simd` of them are resident on
// every CU. The figures price the kernels' instruction counts (rocprofv3 SQ_INSTS_VALU) in time.
// (reference: the autotuner's micro-benchmarks, kangaroo_smat/autotune.cu; no entry point of its own there)
#include "dbk_common.h"

namespace {

typedef float v32f __attribute__((ext_vector_type(32)));

#define DBK_R8(OP) OP(0) OP(1) OP(2) OP(3) OP(4) OP(5) OP(6) OP(7)
#define DBK_R64(OP) DBK_R8(OP) DBK_R8(OP) DBK_R8(OP) DBK_R8(OP) DBK_R8(OP) DBK_R8(OP) DBK_R8(OP) DBK_R8(OP)
#define DBK_OP_ADD(r) "v_add_f32 %" #r ", %" #r ", %8\n\t"
#define DBK_OP_FMA(r) "v_fma_f32 %" #r ", %" #r ", %8, %9\n\t"
#define DBK_OP_MAX(r) "v_max_f32 %" #r ", %" #r ", %8\n\t"
#define DBK_OP_MAX3(r) "v_max3_f32 %" #r ", %" #r ", %8, %9\n\t"
#define DBK_IDX8(g) "v_add_f32 v96, v96, " g "\n\tv_add_f32 v97, v97, " g "\n\tv_add_f32 v98, v98, " g "\n\tv_add_f32 v99, v99, " g "\n\t" \
                    "v_add_f32 v100, v100, " g "\n\tv_add_f32 v101, v101, " g "\n\tv_add_f32 v102, v102, " g "\n\tv_add_f32 v103, v103, " g "\n\t"
#define DBK_IDX64 DBK_IDX8("%2") DBK_IDX8("%3") DBK_IDX8("%2") DBK_IDX8("%3") DBK_IDX8("%2") DBK_IDX8("%3") DBK_IDX8("%2") DBK_IDX8("%3")

template <int KIND>
__global__ __launch_bounds__(256) void k_probe(const float* __restrict__ in, float* __restrict__ out, int iters)
{
    float a[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) a[i] = in[(threadIdx.x + i) & 127];
    const float g0 = in[threadIdx.x & 63], g1 = in[(threadIdx.x & 63) + 64];
    v32f planes;
#pragma unroll
    for (int i = 0; i < 32; ++i) planes[i] = 0.0f;
    const int idx = 8 * (int)(blockIdx.x & 1);                     // wave-uniform register index (index-mode kind)
    for (int i = 0; i < iters; ++i) {
#define DBK_REGS "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7])
        if (KIND == 0) asm volatile(DBK_R64(DBK_OP_ADD) : DBK_REGS : "v"(g0), "v"(g1));
        if (KIND == 1) asm volatile(DBK_R64(DBK_OP_FMA) : DBK_REGS : "v"(g0), "v"(g1));
        if (KIND == 2) asm volatile(DBK_R64(DBK_OP_MAX) : DBK_REGS : "v"(g0), "v"(g1));
        if (KIND == 3) asm volatile(DBK_R64(DBK_OP_MAX3) : DBK_REGS : "v"(g0), "v"(g1));
        if (KIND == 4) asm volatile("s_set_gpr_idx_on %1, 0x9\n\t" DBK_IDX64 "s_set_gpr_idx_off" : "+{v[96:127]}"(planes) : "s"(idx), "v"(g0), "v"(g1));
#undef DBK_REGS
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += a[i];
#pragma unroll
    for (int i = 0; i < 32; ++i) s += planes[i];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace

extern "C" int dbk_probe_valu_issue(int kind, int waves_per_simd, int iters, double* ginstr_per_s_per_simd)
{
    DBK_CHECK(kind >= 0 && kind <= 4, "ValueError: kind must be 0 (add), 1 (fma), 2 (max), 3 (max3) or 4 (index-mode add)");
    DBK_CHECK(waves_per_simd >= 1 && waves_per_simd <= 8 && iters >= 1 && ginstr_per_s_per_simd, "ValueError: bad probe arguments");
    int dev = 0, ncu = 0;
    DBK_HIP(hipGetDevice(&dev));
    DBK_HIP(hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, dev));
    const unsigned nblock = (unsigned)ncu * (unsigned)waves_per_simd;
    float *in = nullptr, *out = nullptr;
    DBK_HIP(hipMalloc(&in, 128 * sizeof(float)));
    DBK_HIP(hipMalloc(&out, (size_t)nblock * 256 * sizeof(float)));
    DBK_HIP(hipMemset(in, 0, 128 * sizeof(float)));
    hipEvent_t e0, e1;
    DBK_HIP(hipEventCreate(&e0));
    DBK_HIP(hipEventCreate(&e1));
    float best = 0.0f;
    for (int rep = 0; rep < 3; ++rep) {                            // the first run warms the clocks up
        DBK_HIP(hipEventRecord(e0, nullptr));
        switch (kind) {
        case 0: hipLaunchKernelGGL(k_probe<0>, dim3(nblock), dim3(256), 0, nullptr, in, out, iters); break;
        case 1: hipLaunchKernelGGL(k_probe<1>, dim3(nblock), dim3(256), 0, nullptr, in, out, iters); break;
        case 2: hipLaunchKernelGGL(k_probe<2>, dim3(nblock), dim3(256), 0, nullptr, in, out, iters); break;
        case 3: hipLaunchKernelGGL(k_probe<3>, dim3(nblock), dim3(256), 0, nullptr, in, out, iters); break;
        default: hipLaunchKernelGGL(k_probe<4>, dim3(nblock), dim3(256), 0, nullptr, in, out, iters); break;
        }
        DBK_HIP(hipEventRecord(e1, nullptr));
        DBK_HIP(hipEventSynchronize(e1));
        float ms = 0.0f;
        DBK_HIP(hipEventElapsedTime(&ms, e0, e1));
        if (rep == 0 || ms < best) best = ms;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(in);
    (void)hipFree(out);
    // wave-instructions per SIMD: each of the CU's four SIMDs runs waves_per_simd waves of iters * 64 instructions
    *ginstr_per_s_per_simd = (double)iters * 64.0 * waves_per_simd / ((double)best * 1e-3) / 1e9;
    dbk::clear_error();
    return 0;
}
