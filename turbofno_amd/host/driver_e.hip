// Drivers TurboFNO_1D_E / TurboFNO_2D_E: the unfused LIBRARY baseline of the spectral layer.
// hipFFT and hipBLAS are called directly (no compatibility shim); the truncation and zero-padding between
// the library calls are two small copy kernels. This executable is a comparator: nothing in libturbofno.so
// depends on it and it is never part of the fused path's timed region.
//
// Step sequence of the reference's baseline (fusion_variants/1D_E_baseline/fused.cu:178-190,
// fusion_variants/2D_E_baseline/fused_trunc_2D.cu:200-227): batched C2C FFT -> keep the first 64 modes per
// transformed axis -> CGEMM (alpha, beta, lda = M, ldb = K, ldc = M) -> zero-pad -> second batched FFT.
// The reference executes its second transform with the FORWARD flag (1D_E.../fused.cu:190); the inverse is what
// is meant, and BACKWARD (unnormalised) is what is executed here. Its 2D result label reads "1D_E"
// (2D_E.../fused_trunc_2D.cu:260); the label printed here is "2D_E".
#include "TurboFNO.h"
#include "utils.h"
#include "inputs.h"
#include <hipblas/hipblas.h>
#include <hipfft/hipfft.h>
#include <cmath>
#include <cstring>

#ifndef TURBOFNO_VARIANT_2D
#define TURBOFNO_VARIANT_2D 0
#endif
#ifndef DEFAULT_CONFIG_PATH
#define DEFAULT_CONFIG_PATH "benchmark_config/problem_size_1d.txt"
#endif


// spec[img][DX][DY] -> A[img][keepx][64]: first 64 modes along Y, first keepx modes along X (keepx = 1 rows of
// a 1D problem are handled by DX = 1). One thread per retained mode pair (float4 = 2 complex).
__global__ void keep_low_modes(const float4* __restrict__ spec, float4* __restrict__ A, long nimg, int DX, int DY, int keepx)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;          // over nimg * keepx * 32
    if (idx >= nimg * keepx * 32) return;
    const int q2 = (int)(idx % 32);
    const long row = idx / 32;                                             // img * keepx + p
    const long img = row / keepx;
    const int p = (int)(row % keepx);
    A[idx] = spec[(img * DX + p) * (DY / 2) + q2];
}

// C[img][keepx][64] -> padded[img][DX][DY], zero outside the retained block. One thread per float4 of the output.
__global__ void pad_low_modes(const float4* __restrict__ C, float4* __restrict__ padded, long nimg, int DX, int DY, int keepx)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;          // over nimg * DX * DY/2
    if (idx >= nimg * DX * (DY / 2)) return;
    const int y2 = (int)(idx % (DY / 2));
    const long row = idx / (DY / 2);
    const long img = row / DX;
    const int p = (int)(row % DX);
    padded[idx] = (p < keepx && y2 < 32) ? C[(img * keepx + p) * 32 + y2] : make_float4(0.f, 0.f, 0.f, 0.f);
}

struct Problem { int bs, dx, dy, n, k; };

#define CHECK_FFT(call)  do { hipfftResult r_ = (call); if (r_ != HIPFFT_SUCCESS) { fprintf(stderr, "hipFFT error %d at %s:%d\n", (int)r_, __FILE__, __LINE__); exit(EXIT_FAILURE); } } while (0)
#define CHECK_BLAS(call) do { hipblasStatus_t r_ = (call); if (r_ != HIPBLAS_STATUS_SUCCESS) { fprintf(stderr, "hipBLAS error %d at %s:%d\n", (int)r_, __FILE__, __LINE__); exit(EXIT_FAILURE); } } while (0)

int main(int argc, char** argv)
{
    // kernel arguments in device memory (ROCm runtime knob, read when HIP initialises; an existing setting wins):
    // about a microsecond less at the start of every kernel
    setenv("HIP_FORCE_DEV_KERNARG", "1", 0);
    std::vector<Problem> problems;
    if (argc == 6) problems.push_back({ atoi(argv[1]), atoi(argv[2]), atoi(argv[3]), atoi(argv[4]), atoi(argv[5]) });
    else {
        auto cfg = load_problem_config(argc == 2 ? argv[1] : DEFAULT_CONFIG_PATH);
        for (int bs : cfg["bs_list"])
            for (int dx : cfg[TURBOFNO_VARIANT_2D ? "DX_list" : "dimX_list"])
                for (int dy : cfg["DY_list"])
                    for (int n : cfg["N_list"])
                        for (int k : cfg["K_list"]) problems.push_back({ bs, dx, dy, n, k });
    }
    if (const char* e = getenv("TURBOFNO_NTEST")) ntest = atoi(e) > 0 ? atoi(e) : ntest;
    hipblasHandle_t blas;
    CHECK_BLAS(hipblasCreate(&blas));
    const float2 alpha = make_float2(1.0f, -1.0f), beta = make_float2(-1.0f, 1.0f);

    for (const Problem& p : problems) {
        // 1D: nimg = bs*dimX signals per channel of length DY (DX plays no role: one row per signal)
        // 2D: nimg = bs images per channel of DX x DY
        const int DX = TURBOFNO_VARIANT_2D ? p.dx : 1, keepx = TURBOFNO_VARIANT_2D ? THREADBLOCK_M : 1;
        const long per_channel = TURBOFNO_VARIANT_2D ? (long)p.bs : (long)p.bs * p.dx;
        const long nin = per_channel * p.k, nout = per_channel * p.n;
        const long M = per_channel * keepx * THREADBLOCK_M;
        const size_t in_elems = (size_t)nin * DX * p.dy, out_elems = (size_t)nout * DX * p.dy;
        const size_t big = in_elems > out_elems ? in_elems : out_elems;
        if (getenv("TURBOFNO_DIGEST")) srand(1);   // same inputs in every executable, whatever the libraries drew from rand()
        const InputKind kind = input_kind_from_name(getenv("TURBOFNO_INPUTS"));
        const uint64_t seed = getenv("TURBOFNO_SEED") ? strtoull(getenv("TURBOFNO_SEED"), nullptr, 0) : default_seed(kind);
        const bool seeded = kind != InputKind::reference_rand;
        const std::vector<float> hx = seeded ? generate_inputs(kind, seed, p.k, per_channel * DX, TURBOFNO_VARIANT_2D ? p.dx : 0, p.dy) : draw_random(2 * in_elems);
        const std::vector<float> hw = seeded ? generate_weights(kind, seed, p.k, p.n) : draw_random(2 * (size_t)p.k * p.n);
        float2 *dx = nullptr, *dspec = nullptr, *dA = nullptr, *dW = nullptr, *dC = nullptr, *dy = nullptr;
        HIP_RT_CALL(hipMalloc(&dx, sizeof(float2) * in_elems));
        HIP_RT_CALL(hipMalloc(&dspec, sizeof(float2) * big));
        HIP_RT_CALL(hipMalloc(&dy, sizeof(float2) * out_elems));
        HIP_RT_CALL(hipMalloc(&dA, sizeof(float2) * M * p.k));
        HIP_RT_CALL(hipMalloc(&dC, sizeof(float2) * M * p.n));
        HIP_RT_CALL(hipMalloc(&dW, sizeof(float2) * p.k * p.n));
        upload_tiled(dx, 2 * in_elems, hx);
        upload_tiled(dW, 2 * (size_t)p.k * p.n, hw);
        HIP_RT_CALL(hipMemset(dC, 0, sizeof(float2) * M * p.n));

        hipfftHandle plan_in, plan_out;
        if (TURBOFNO_VARIANT_2D) {
            int dims[2] = { p.dx, p.dy };
            CHECK_FFT(hipfftPlanMany(&plan_in, 2, dims, nullptr, 1, p.dx * p.dy, nullptr, 1, p.dx * p.dy, HIPFFT_C2C, (int)nin));
            CHECK_FFT(hipfftPlanMany(&plan_out, 2, dims, nullptr, 1, p.dx * p.dy, nullptr, 1, p.dx * p.dy, HIPFFT_C2C, (int)nout));
        } else {
            CHECK_FFT(hipfftPlan1d(&plan_in, p.dy, HIPFFT_C2C, (int)nin));
            CHECK_FFT(hipfftPlan1d(&plan_out, p.dy, HIPFFT_C2C, (int)nout));
        }
        auto launch = [&]() {
            CHECK_FFT(hipfftExecC2C(plan_in, (hipfftComplex*)dx, (hipfftComplex*)dspec, HIPFFT_FORWARD));
            const long keep_threads = nin * keepx * 32;
            hipLaunchKernelGGL(keep_low_modes, dim3((unsigned)((keep_threads + 255) / 256)), dim3(256), 0, 0,
                               (const float4*)dspec, (float4*)dA, nin, DX, p.dy, keepx);
            CHECK_BLAS(hipblasCgemm(blas, HIPBLAS_OP_N, HIPBLAS_OP_N, (int)M, p.n, p.k, &alpha, dA, (int)M,
                                    dW, p.k, &beta, dC, (int)M));
            const long pad_threads = nout * DX * (p.dy / 2);
            hipLaunchKernelGGL(pad_low_modes, dim3((unsigned)((pad_threads + 255) / 256)), dim3(256), 0, 0,
                               (const float4*)dC, (float4*)dspec, nout, DX, p.dy, keepx);
            CHECK_FFT(hipfftExecC2C(plan_out, (hipfftComplex*)dspec, (hipfftComplex*)dy, HIPFFT_BACKWARD));
        };
        HIP_RT_CALL(hipDeviceSynchronize());
        launch();
        CHECK_HIP_KERNEL();
        HIP_RT_CALL(hipDeviceSynchronize());
        if (getenv("TURBOFNO_DIGEST")) print_output_digest(dy, out_elems);
        HIP_RT_CALL(hipMemset(dC, 0, sizeof(float2) * M * p.n));

        hipEvent_t t_begin, t_end;
        float elapsed_time = 0.f;
        HIP_RT_CALL(hipEventCreate(&t_begin));
        HIP_RT_CALL(hipEventCreate(&t_end));
        HIP_RT_CALL(hipEventRecord(t_begin));
        for (int i = 0; i < ntest; ++i) {
            launch();
            HIP_RT_CALL(hipDeviceSynchronize());
        }
        HIP_RT_CALL(hipEventRecord(t_end));
        HIP_RT_CALL(hipEventSynchronize(t_end));
        HIP_RT_CALL(hipEventElapsedTime(&elapsed_time, t_begin, t_end));
        elapsed_time /= ntest;
        if (TURBOFNO_VARIANT_2D)
            printf("2D_E, bs=%-4d, DX=%-4d, DY=%-4d, N=%-4d, K=%-4d, TIME=%8.3fms\n", p.bs, p.dx, p.dy, p.n, p.k, elapsed_time);
        else
            printf("1D_E, bs=%-4d, dimX=%-4d, DY=%-4d, N=%-4d, K=%-4d, TIME=%8.3fms\n", p.bs, p.dx, p.dy, p.n, p.k, elapsed_time);
        fflush(stdout);
        if (getenv("TURBOFNO_STATS")) print_iteration_stats(launch, ntest);
        CHECK_FFT(hipfftDestroy(plan_in));
        CHECK_FFT(hipfftDestroy(plan_out));
        HIP_RT_CALL(hipEventDestroy(t_begin)); HIP_RT_CALL(hipEventDestroy(t_end));
        HIP_RT_CALL(hipFree(dx)); HIP_RT_CALL(hipFree(dspec)); HIP_RT_CALL(hipFree(dy));
        HIP_RT_CALL(hipFree(dA)); HIP_RT_CALL(hipFree(dC)); HIP_RT_CALL(hipFree(dW));

    }
    CHECK_BLAS(hipblasDestroy(blas));
    return 0;
}
