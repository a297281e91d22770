// Drivers TurboFNO_{1D,2D}_{A,B,C,D}: the spectral layer built from separately launched stages (A), with the
// forward transform fused into the GEMM (B), with the backward transform fused into the GEMM (C), and fully
// fused (D), each timed per problem. One source, selected by TURBOFNO_VARIANT / TURBOFNO_VARIANT_2D.
// Stage sequences follow the reference's mains: 1D_A.../fused.cu:195-203, 1D_B.../fused.cu:141-144,
// 1D_C.../fused.cu:139-144, 2D_A.../fused_trunc_2D.cu:189-219, 2D_B...:183-197, 2D_C...:184-199.
//
// Surface kept from the reference (fusion_variants/1D_D_exp_fused_fft_cgemm_ifft/fused.cu:20-151,
// fusion_variants/2D_D_exp_fused_fft_cgemm_ifft/fused_trunc_2D.cu:33-208):
//   * problems come from benchmark_config/problem_size_{1d,2d}.txt (DEFAULT_CONFIG_PATH baked in at
//     build time), loop order bs -> dimX|DX -> DY -> N -> K;
//   * alternatively five positional integers "<bs> <dimX|DX> <DY> <N> <K>" run a single problem
//     (fusion_variants_benchmark/1D_D_exp_fused_fft_cgemm_ifft/fused.cu:33-46), or one argument
//     names another config file (documented at README.md:122-132);
//   * inputs: +-{0..9}e-3 from rand(); alpha = (1,-1), beta = (-1,1) on a zeroed C (variants A and B use beta);
//   * timing: one warm-up, then ntest x (launch + device synchronise) between two events, mean;
//   * one result line per problem, format identical to fused.cu:146-147 / fused_trunc_2D.cu:203-204.
// Differences: device buffers are sized per problem (the reference allocates once for its largest
// hard-coded problem); the kernels are reached through the C ABI of include/turbofno.h.
#include "../../include/turbofno.h"
#include "TurboFNO.h"
#include "utils.h"
#include "inputs.h"
#include <cmath>
#include <cstring>
#include <string>

#ifndef TURBOFNO_VARIANT_2D
#define TURBOFNO_VARIANT_2D 0
#endif
#ifndef TURBOFNO_VARIANT
#define TURBOFNO_VARIANT 'D'
#endif
#ifndef DEFAULT_CONFIG_PATH
#define DEFAULT_CONFIG_PATH "benchmark_config/problem_size_1d.txt"
#endif

struct Problem { int bs, dx, dy, n, k; };

// a positional argument as a positive integer; anything else (text, trailing characters, zero, overflow) ends the run
static int positive_int(const char* text, const char* name)
{
    char* end = nullptr;
    const long v = strtol(text, &end, 10);
    if (end == text || *end != '\0' || v <= 0 || v > 0x7fffffffL) {
        fprintf(stderr, "argument %s = \"%s\" is not a positive integer\n", name, text);
        exit(EXIT_FAILURE);
    }
    return (int)v;
}

// log2 of a transform length the kernels are built for (128 ... 1024), or -1
static int log2_of_length(int v)
{
    for (int l = 7; l <= 10; ++l)
        if (v == (1 << l)) return l;
    return -1;
}

static std::vector<Problem> problems_from(int argc, char** argv)
{
    std::vector<Problem> out;
    if (argc == 6) {
        out.push_back({ positive_int(argv[1], "bs"), positive_int(argv[2], TURBOFNO_VARIANT_2D ? "DX" : "dimX"),
                        positive_int(argv[3], "DY"), positive_int(argv[4], "N"), positive_int(argv[5], "K") });
        return out;
    }
    auto cfg = load_problem_config(argc == 2 ? argv[1] : DEFAULT_CONFIG_PATH);
    const char* xkey = TURBOFNO_VARIANT_2D ? "DX_list" : "dimX_list";
    for (int bs : cfg["bs_list"])
        for (int dx : cfg[xkey])
            for (int dy : cfg["DY_list"])
                for (int n : cfg["N_list"])
                    for (int k : cfg["K_list"]) out.push_back({ bs, dx, dy, n, k });
    return out;
}

int main(int argc, char** argv)
{
    // kernel arguments in device memory (ROCm runtime knob, read when HIP initialises; an existing setting wins):
    // about a microsecond less at the start of every kernel
    setenv("HIP_FORCE_DEV_KERNARG", "1", 0);
    const float alpha_re = 1.0f, alpha_im = -1.0f;
    int algo = TURBOFNO_2D_AUTO;
    if (const char* e = getenv("TURBOFNO_2D_ALGO")) algo = atoi(e);
    if (const char* e = getenv("TURBOFNO_NTEST")) ntest = atoi(e) > 0 ? atoi(e) : ntest;
    // measurement aid of these executables only (the library itself reads no environment): forces one of the fused 1D kernels
    if (const char* e = getenv("TURBOFNO_1D_ALGO")) CHECK_TURBOFNO(turbofno_set_1d_algo(atoi(e)));

    const std::vector<Problem> problems = problems_from(argc, argv);     // argument errors end the run before any HIP call

    // Like every other buffer of the run, the exchange memory of the clustered 1D kernel (small grids with 64 channels or
    // more) belongs to this main: allocated once, attached to the default stream, which all launches below use.
    // TURBOFNO_NO_EXCHANGE=1 leaves it out (the library then runs kernels that need none).
    void* exchange = nullptr;
    if (TURBOFNO_VARIANT == 'D' && !getenv("TURBOFNO_NO_EXCHANGE")) {
        const size_t bytes = turbofno_exchange_bytes(0);
        HIP_RT_CALL(hipMalloc(&exchange, bytes));
        if (exchange) CHECK_TURBOFNO(turbofno_exchange_attach(nullptr, exchange, bytes));
    }

    for (const Problem& p : problems) {
        if (p.k % THREADBLOCK_K != 0) { fprintf(stderr, "K=%d is not a multiple of %d: problem skipped\n", p.k, THREADBLOCK_K); continue; }
        if (p.bs <= 0 || p.dx <= 0 || p.n <= 0 || p.k <= 0 || p.n % THREADBLOCK_M != 0) {
            fprintf(stderr, "bs=%d, %s=%d, N=%d, K=%d: sizes must be positive and N a multiple of %d: problem skipped\n", p.bs,
                    TURBOFNO_VARIANT_2D ? "DX" : "dimX", p.dx, p.n, p.k, THREADBLOCK_M);
            continue;
        }
        // transform lengths index the kernel tables by log2(length) - 7: only exact powers of two from 128 to 1024 have an
        // entry (a rounded logarithm would run a kernel of another length on these buffers)
        const int logDY = log2_of_length(p.dy), logDX = TURBOFNO_VARIANT_2D ? log2_of_length(p.dx) : 0;
        if (logDY < 0 || logDX < 0) {
            fprintf(stderr, "DY=%d%s: transform lengths must be 128, 256, 512 or 1024: problem skipped\n", p.dy,
                    TURBOFNO_VARIANT_2D ? (", DX=" + std::to_string(p.dx)).c_str() : "");
            continue;
        }
        // 1D: x[K][bs*dimX][DY]; 2D: x[K][bs][DX][DY]
        const size_t per_channel = TURBOFNO_VARIANT_2D ? (size_t)p.bs * p.dx * p.dy : (size_t)p.bs * p.dx * p.dy;
        const size_t in_elems = per_channel * p.k, out_elems = per_channel * p.n, w_elems = (size_t)p.k * p.n;
        if (getenv("TURBOFNO_DIGEST")) srand(1);   // same inputs in every executable, whatever the libraries drew from rand()
        // inputs: the reference's rand() fill, or (TURBOFNO_INPUTS) one of the seeded distributions of the benchmark configurations
        const InputKind kind = input_kind_from_name(getenv("TURBOFNO_INPUTS"));
        const uint64_t seed = getenv("TURBOFNO_SEED") ? strtoull(getenv("TURBOFNO_SEED"), nullptr, 0) : default_seed(kind);
        const bool seeded = kind != InputKind::reference_rand;
        const long signals = TURBOFNO_VARIANT_2D ? (long)p.bs * p.dx : (long)p.bs * p.dx;
        const std::vector<float> hx = seeded ? generate_inputs(kind, seed, p.k, signals, TURBOFNO_VARIANT_2D ? p.dx : 0, p.dy) : draw_random(2 * in_elems);
        const std::vector<float> hw = seeded ? generate_weights(kind, seed, p.k, p.n) : draw_random(2 * w_elems);
        void *dx = nullptr, *dw = nullptr, *dy = nullptr, *dws = nullptr;
        HIP_RT_CALL(hipMalloc(&dx, sizeof(float) * 2 * in_elems));
        HIP_RT_CALL(hipMalloc(&dw, sizeof(float) * 2 * w_elems));
        HIP_RT_CALL(hipMalloc(&dy, sizeof(float) * 2 * out_elems));
        upload_tiled(dx, 2 * in_elems, hx);
        upload_tiled(dw, 2 * w_elems, hw);
        size_t ws_bytes = 0;
        if (TURBOFNO_VARIANT_2D && TURBOFNO_VARIANT == 'D') {
            ws_bytes = turbofno_layer_2d_workspace_bytes(p.bs, p.dx, p.dy, p.k, p.n, algo);
            HIP_RT_CALL(hipMalloc(&dws, ws_bytes ? ws_bytes : 256));
        }
        // stage buffers of the unfused / half-fused variants: A[M x K], C[M x N] and, in 2D, the X-stage
        // intermediates t1[K*bs][64][DY], t2[N*bs][64][DY]
        const long S = TURBOFNO_VARIANT_2D ? (long)p.bs * THREADBLOCK_M : (long)p.bs * p.dx;   // signals per channel of the Y stage
        const long M = THREADBLOCK_M * S;
        void *dA = nullptr, *dC = nullptr, *t1 = nullptr, *t2 = nullptr;
        if (TURBOFNO_VARIANT != 'D') {
            HIP_RT_CALL(hipMalloc(&dA, sizeof(float) * 2 * M * p.k));
            HIP_RT_CALL(hipMalloc(&dC, sizeof(float) * 2 * M * p.n));
            HIP_RT_CALL(hipMemset(dC, 0, sizeof(float) * 2 * M * p.n));
            if (TURBOFNO_VARIANT_2D) {
                HIP_RT_CALL(hipMalloc(&t1, sizeof(float) * 2 * S * p.dy * p.k));
                HIP_RT_CALL(hipMalloc(&t2, sizeof(float) * 2 * S * p.dy * p.n));
            }
        }
        const float beta_re = -1.0f, beta_im = 1.0f;
        auto launch = [&]() {
            const void* yin = dx;            // input of the Y stage
            void* yout = dy;                 // output of the Y stage
            if (TURBOFNO_VARIANT == 'D') {
                if (TURBOFNO_VARIANT_2D)
                    CHECK_TURBOFNO(turbofno_layer_2d(p.bs, p.dx, p.dy, p.k, p.n, dx, dw, dy, alpha_re, alpha_im, dws, ws_bytes, algo, nullptr));
                else
                    CHECK_TURBOFNO(turbofno_layer_1d(p.bs, p.dx, p.dy, p.k, p.n, dx, dw, dy, alpha_re, alpha_im, nullptr));
                return;
            }
            if (TURBOFNO_VARIANT_2D) {
                CHECK_TURBOFNO(turbofno_fft_stride(logDX, dx, t1, threadblock_bs, p.dy, (long)p.dy * p.k * p.bs, THREADBLOCK_M, nullptr));
                yin = t1; yout = t2;
            }
            if (TURBOFNO_VARIANT == 'A') {
                CHECK_TURBOFNO(turbofno_fft_stride_DY(logDY, yin, dA, threadblock_bs, S * p.k, nullptr));
                CHECK_TURBOFNO(turbofno_cgemm(M, p.n, p.k, dA, dw, dC, alpha_re, alpha_im, beta_re, beta_im, nullptr));
                CHECK_TURBOFNO(turbofno_ifft_stride_DY(logDY, dC, yout, threadblock_bs, S * p.n, nullptr));
            } else if (TURBOFNO_VARIANT == 'B') {
                CHECK_TURBOFNO(turbofno_fused_fft_cgemm(logDY, M, p.n, p.k, yin, dw, dC, alpha_re, alpha_im, beta_re, beta_im, nullptr));
                CHECK_TURBOFNO(turbofno_ifft_stride_DY(logDY, dC, yout, threadblock_bs, S * p.n, nullptr));
            } else {
                CHECK_TURBOFNO(turbofno_fft_stride_DY(logDY, yin, dA, threadblock_bs, S * p.k, nullptr));
                CHECK_TURBOFNO(turbofno_fused_cgemm_ifft(logDY, M, p.n, p.k, dA, dw, dC, yout, alpha_re, alpha_im, beta_re, beta_im, nullptr));
            }
            if (TURBOFNO_VARIANT_2D)
                CHECK_TURBOFNO(turbofno_ifft_stride(logDX, t2, dy, threadblock_bs, p.dy, (long)p.dy * p.n * p.bs, THREADBLOCK_M, nullptr));
        };
        HIP_RT_CALL(hipDeviceSynchronize());
        launch();
        CHECK_HIP_KERNEL();
        HIP_RT_CALL(hipDeviceSynchronize());
        CHECK_HIP_KERNEL();
        if (getenv("TURBOFNO_DIGEST")) print_output_digest(dy, out_elems);

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
            printf("2D_%c, bs=%-4d, DX=%-4d, DY=%-4d, N=%-4d, K=%-4d, TIME=%8.3fms\n", TURBOFNO_VARIANT, p.bs, p.dx, p.dy, p.n, p.k, elapsed_time);
        else
            printf("1D_%c, bs=%-4d, dimX=%-4d, DY=%-4d, N=%-4d, K=%-4d, TIME=%8.3fms\n", TURBOFNO_VARIANT, p.bs, p.dx, p.dy, p.n, p.k, elapsed_time);
        fflush(stdout);
        if (getenv("TURBOFNO_STATS")) print_iteration_stats(launch, ntest);
        HIP_RT_CALL(hipEventDestroy(t_begin));
        HIP_RT_CALL(hipEventDestroy(t_end));
        HIP_RT_CALL(hipFree(dx)); HIP_RT_CALL(hipFree(dw)); HIP_RT_CALL(hipFree(dy));
        if (dws) HIP_RT_CALL(hipFree(dws));
        if (dA) HIP_RT_CALL(hipFree(dA));
        if (dC) HIP_RT_CALL(hipFree(dC));
        if (t1) HIP_RT_CALL(hipFree(t1));
        if (t2) HIP_RT_CALL(hipFree(t2));
    }
    if (exchange) {
        unsigned gave_up = 0;
        if (turbofno_exchange_status(nullptr, &gave_up) == TURBOFNO_ERR_EXCHANGE)
            fprintf(stderr, "note: %u cluster member(s) ran out of their wait during this run (results valid, those launches slow)\n", gave_up);
        CHECK_TURBOFNO(turbofno_exchange_detach(nullptr));
        HIP_RT_CALL(hipDeviceSynchronize());
        HIP_RT_CALL(hipFree(exchange));
    }
    return 0;
}
