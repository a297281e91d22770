// Memory-only probes with the access patterns of the layer's kernels: what HBM delivers for these patterns when no
// arithmetic is in the way. The rooflines of the kernels are quoted against the 8 TB/s peak; these figures say how
// much of the distance to that peak belongs to the pattern (and to HBM itself) rather than to a kernel.
//   bin/TurboFNO_hbm_probe            (no arguments; prints one line per probe)
// Every probe is the mean of 20 launches, each between its own pair of events, after one warm-up launch.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>

typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));

#define CHECK(x)                                                                              \
    do {                                                                                      \
        hipError_t e_ = (x);                                                                  \
        if (e_ != hipSuccess) {                                                               \
            fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_)); \
            exit(1);                                                                          \
        }                                                                                     \
    } while (0)

// ---- image pattern: a persistent 1024-thread block per CU walks over 256 x 256 images; a 16-lane group moves one
// ---- row as samples t + 16 i (128 contiguous bytes per instruction and group), as the whole-image 2D kernels do
template <bool STREAMING>
__global__ __launch_bounds__(1024) void image_store(float2* y, int nimg, float s)
{
    const int grp = threadIdx.x >> 4, t = threadIdx.x & 15;
    for (int img = blockIdx.x; img < nimg; img += gridDim.x) {
        float2* base = y + (size_t)img * 65536;
        for (int rr = 0; rr < 4; ++rr) {
            float2* row = base + (size_t)(grp + 64 * rr) * 256;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                v2f q = { s + i, s - t };
                if (STREAMING) __builtin_nontemporal_store(q, reinterpret_cast<v2f*>(row + t + 16 * i));
                else row[t + 16 * i] = make_float2(q.x, q.y);
            }
        }
    }
}

template <bool STREAMING>
__global__ __launch_bounds__(1024) void image_load(const float2* x, float* sink, int nimg)
{
    const int grp = threadIdx.x >> 4, t = threadIdx.x & 15;
    float acc = 0.f;
    for (int img = blockIdx.x; img < nimg; img += gridDim.x) {
        const float2* base = x + (size_t)img * 65536;
        for (int rr = 0; rr < 4; ++rr) {
            const float2* row = base + (size_t)(grp + 64 * rr) * 256;
            float2 v[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                if (STREAMING) {
                    const v2f q = __builtin_nontemporal_load(reinterpret_cast<const v2f*>(row + t + 16 * i));
                    v[i] = make_float2(q.x, q.y);
                } else {
                    v[i] = row[t + 16 * i];
                }
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) acc += v[i].x + v[i].y;
        }
    }
    if (acc == 1.2345f) sink[threadIdx.x] = acc;      // keeps the loads alive
}

// ---- linear fill: every thread writes 16 bytes, the grid sweeps the buffer as one front
__global__ void linear_fill(v4f* p, size_t total, float s)
{
    const v4f q = { s, s, s, s + threadIdx.x };
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) p[i] = q;
}

// ---- fused 1D layer pattern, DY = 256: item s reads K rows of 2 KiB that lie S rows apart and writes N such rows;
// ---- one wavefront per item, a 16-lane group per row
template <bool STREAMING_STORES>
__global__ __launch_bounds__(64) void layer1d_pattern(const float2* __restrict__ x, float2* __restrict__ y, int S, int K, int N)
{
    const int lane = threadIdx.x, g = lane >> 4, t = lane & 15;
    const long s = blockIdx.x;
    float2 acc = make_float2(0.f, 0.f);
    for (int kc = 0; kc < K; kc += 4) {
        const float2* src = x + ((long)(kc + g) * S + s) * 256 + t;
        float2 v[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = src[16 * i];
#pragma unroll
        for (int i = 0; i < 16; ++i) { acc.x += v[i].x; acc.y += v[i].y; }
    }
    for (int n = 0; n < N; n += 4) {
        float2* dst = y + ((long)(n + g) * S + s) * 256 + t;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            v2f q = { acc.x + i, acc.y };
            if (STREAMING_STORES) __builtin_nontemporal_store(q, reinterpret_cast<v2f*>(dst + 16 * i));
            else dst[16 * i] = make_float2(q.x, q.y);
        }
    }
}

int main()
{
    const int nimg = 1024, S = 4096, K = 32, N = 64;
    const size_t img_bytes = (size_t)nimg * 65536 * 8;                    // 512 MiB
    float2 *a, *b;
    float* sink;
    CHECK(hipMalloc(&a, img_bytes));
    CHECK(hipMalloc(&b, img_bytes));
    CHECK(hipMalloc(&sink, 4096));
    CHECK(hipMemset(a, 0, img_bytes));
    CHECK(hipMemset(b, 0, img_bytes));
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    // `before` runs ahead of every timed launch, outside the timed span (used to push the data out of the caches)
    auto run = [&](const char* name, double bytes, auto launch, auto before) {
        before();
        launch();
        CHECK(hipDeviceSynchronize());
        double total_ms = 0;
        for (int r = 0; r < 20; ++r) {
            before();
            CHECK(hipEventRecord(e0));
            launch();
            CHECK(hipEventRecord(e1));
            CHECK(hipEventSynchronize(e1));
            float ms;
            CHECK(hipEventElapsedTime(&ms, e0, e1));
            total_ms += ms;
        }
        const double ms = total_ms / 20;
        printf("%-64s %8.1f us %7.0f GB/s  %.3f of 8 TB/s\n", name, ms * 1e3, bytes / ms / 1e6, bytes / ms / 1e6 / 8000.0);
    };
    auto nothing = [] {};
    auto flush = [&] { hipLaunchKernelGGL(linear_fill, dim3(cus), dim3(256), 0, 0, reinterpret_cast<v4f*>(b), img_bytes / 16, 2.f); };
    printf("device: %s, %d CUs\n", prop.name, cus);
    // each read probe follows an untimed 512 MiB fill of the OTHER buffer, so that the data it reads is not cache resident
    run("image pattern, store only, streaming stores (512 MiB)", (double)img_bytes,
        [&] { hipLaunchKernelGGL(image_store<true>, dim3(cus), dim3(1024), 0, 0, a, nimg, 1.f); }, nothing);
    run("image pattern, store only, plain stores (512 MiB)", (double)img_bytes,
        [&] { hipLaunchKernelGGL(image_store<false>, dim3(cus), dim3(1024), 0, 0, a, nimg, 1.f); }, nothing);
    run("image pattern, load only, streaming loads (512 MiB)", (double)img_bytes,
        [&] { hipLaunchKernelGGL(image_load<true>, dim3(cus), dim3(1024), 0, 0, a, sink, nimg); }, flush);
    run("image pattern, load only, plain loads (512 MiB)", (double)img_bytes,
        [&] { hipLaunchKernelGGL(image_load<false>, dim3(cus), dim3(1024), 0, 0, a, sink, nimg); }, flush);
    run("linear fill, 256 threads per CU (512 MiB)", (double)img_bytes,
        [&] { hipLaunchKernelGGL(linear_fill, dim3(cus), dim3(256), 0, 0, reinterpret_cast<v4f*>(b), img_bytes / 16, 2.f); }, nothing);
    run("linear fill, 1024 threads per CU (512 MiB)", (double)img_bytes,
        [&] { hipLaunchKernelGGL(linear_fill, dim3(cus), dim3(1024), 0, 0, reinterpret_cast<v4f*>(b), img_bytes / 16, 2.f); }, nothing);
    run("hipMemsetAsync (512 MiB)", (double)img_bytes, [&] { CHECK(hipMemsetAsync(b, 1, img_bytes, 0)); }, nothing);
    run("hipMemcpyAsync device to device (512 MiB read + 512 MiB written)", 2.0 * img_bytes,
        [&] { CHECK(hipMemcpyAsync(b, a, img_bytes, hipMemcpyDeviceToDevice, 0)); }, nothing);
    const double b1d = (double)(K + N) * S * 2048;
    run("1D layer pattern bs=4096 DY=256 K=32 N=64, plain stores", b1d,
        [&] { hipLaunchKernelGGL(layer1d_pattern<false>, dim3(S), dim3(64), 0, 0, a, b, S, K, N); }, nothing);
    run("1D layer pattern bs=4096 DY=256 K=32 N=64, streaming stores", b1d,
        [&] { hipLaunchKernelGGL(layer1d_pattern<true>, dim3(S), dim3(64), 0, 0, a, b, S, K, N); }, nothing);
    CHECK(hipGetLastError());
    return 0;
}
