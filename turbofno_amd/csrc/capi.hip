// C ABI of the library: argument validation, dispatch by transform length, error strings.
// Declarations and the reference interfaces each entry point replaces are in include/turbofno.h.
#include "../../include/turbofno.h"
#include "kernels.h"
#include <atomic>
#include <cstdarg>
#include <cstdio>

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_status(hipError_t e, const char* what)
{
    if (e == hipSuccess) return TURBOFNO_OK;
    return fail(TURBOFNO_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

int log2_exact(long v)
{
    if (v <= 0 || (v & (v - 1))) return -1;
    int l = 0;
    while ((1L << l) < v) ++l;
    return l;
}

bool length_built(int logD) { return logD >= 7 && logD <= 10; }          // 1D kernels and the X-axis kernels
bool image_length_built(int logD) { return logD == 7 || logD == 8; }    // rows of an image that one block holds
// the whole-image path of the 2D layer also takes DX of 512 and 1024, as two or four decimated parts of 256 rows
bool whole_image_built(int DX, int DY) { return length_built(log2_exact(DX)) && length_built(log2_exact(DY)); }
int image_parts(int DX) { return DX > 256 ? DX / 256 : 1; }

int check_gemm_dims(long M, int N, int K)
{
    if (M <= 0 || N <= 0 || K <= 0) return fail(TURBOFNO_ERR_INVALID_ARG, "M, N, K must be positive (M=%ld N=%d K=%d)", M, N, K);
    if (M % 64) return fail(TURBOFNO_ERR_INVALID_ARG, "M=%ld is not a multiple of 64 (64 retained modes per signal)", M);
    if (N % 64) return fail(TURBOFNO_ERR_INVALID_ARG, "N=%d is not a multiple of the 64-wide output tile", N);
    if (K % 8) return fail(TURBOFNO_ERR_INVALID_ARG, "K=%d is not a multiple of the 8-deep K tile", K);
    return TURBOFNO_OK;
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

// AUTO: the whole-image path runs one persistent block per image and moves 2/3 of the bytes of the three-kernel path,
// which in turn spreads an image over many blocks and gets three short launches through sooner when there are few
// images. Measured on MI355X (256 CUs; 160 shapes, both paths back to back): from a batch of 8 the whole-image path is
// ahead (by up to 2x at bs = 16) but for two groups of shapes (below); with a batch of 4 to 7 it is ahead for 256 x 256
// images once (K + N) * bs reaches 768 images in and out, and for 128 x 256 images with N >= 128; below a batch of 4 the
// three-kernel path is 12-100 % ahead everywhere.
int pick_algo(int bs, int DX, int DY, int K, int N, int algo)
{
    if (algo != TURBOFNO_2D_AUTO) return algo;
    if (DX > 256 || DY > 256) {
        // Long axes on the whole-image kernels (512 / 1024 rows as interleaved parts of 256, rows of 512 / 1024 with 32 /
        // 64 lanes each): x and y move once and nothing but 64 x 64 modes in between, against intermediates of 1/8 (length
        // 512) or 1/16 (1024) of the data, twice over, for three stages; but one block per part of an image needs enough
        // of them. Measured on MI355X (348 shapes, bs 1-32, all three paths back to back): ahead from the volume of
        // input and output below, by 3-10 % there and by 13-34 % at several GiB (3 GiB of 512 x 512: 752 -> 600 us);
        // behind by up to 2x on small problems.
        static const int whole_from_mib[4][4] = {       // [log2 DX - 7][log2 DY - 7]
            { 0, 0, 576, 4608 }, { 0, 0, 768, 3072 }, { 576, 576, 768, 2560 }, { 1152, 1280, 2560, 4608 } };
        const long mib = ((long)K + N) * bs * DX * DY >> 17;
        const int lx = log2_exact(DX) - 7, ly = log2_exact(DY) - 7;
        if (lx >= 0 && lx < 4 && ly >= 0 && ly < 4 && mib >= whole_from_mib[lx][ly]) return TURBOFNO_2D_WHOLE_IMAGE;
    }
    if (DX > 256 || DY > 256) {
        // otherwise three stages. The axis that is transformed first is the one whose
        // truncation shrinks the intermediates most, i.e. the longer one (DY = 4 DX: half the time of the other order;
        // DX = 4 DY: the reverse). Square images: whole rows first (9-18 % ahead) unless the grid is small.
        if (DY != DX) return DY > DX ? TURBOFNO_2D_ROWS_FIRST : TURBOFNO_2D_THREE_KERNEL;
        return (DY >= 1024 || (long)K * bs >= 128) ? TURBOFNO_2D_ROWS_FIRST : TURBOFNO_2D_THREE_KERNEL;
    }
    if (bs >= 16) return TURBOFNO_2D_WHOLE_IMAGE;
    if (bs < 4) return TURBOFNO_2D_THREE_KERNEL;
    const bool big = DX == 256 && DY == 256;
    if (bs >= 8) {
        // two exceptions measured 7-15 % behind: few images of 256 x 256, and rows of 128 with 64 output channels
        if (big && ((long)K + N) * bs < 768) return TURBOFNO_2D_THREE_KERNEL;
        if (DY == 128 && N == 64 && K < 128) return TURBOFNO_2D_THREE_KERNEL;
        return TURBOFNO_2D_WHOLE_IMAGE;
    }
    if (big && ((long)K + N) * bs >= 768) return TURBOFNO_2D_WHOLE_IMAGE;
    if (DX == 128 && DY == 256 && N >= 128) return TURBOFNO_2D_WHOLE_IMAGE;
    return TURBOFNO_2D_THREE_KERNEL;
}

}  // namespace

extern "C" {

int turbofno_abi_version(void) { return 2; }

const char* turbofno_last_error_string(void) { return g_err; }

// The fused 1D entry point keeps the reference's kernel signature, which has no room for an algorithm selector:
// the process-wide selector set by turbofno_set_1d_algo (0 by size, 1 SIMT contraction, 2 / 3 matrix cores with
// 512- / 256-thread blocks, 4 matrix cores with 512 threads and 32-channel output tiles, 5 matrix cores with one
// wavefront per signal set and output tile, 6 matrix cores with the K channels of an item split over the waves of a
// block, 7 matrix cores with the K channels of a signal set split over a cluster of blocks, 8 matrix cores with tiles of
// 128 output channels) overrides the choice by size.
static std::atomic<int> g_algo_1d{ 0 };
static int algo_1d() { return g_algo_1d.load(std::memory_order_relaxed); }

int turbofno_set_1d_algo(int algo)
{
    if (algo < 0 || algo > TURBOFNO_1D_ALGO_MAX) return fail(TURBOFNO_ERR_INVALID_ARG, "1D algo %d outside 0..%d", algo, TURBOFNO_1D_ALGO_MAX);
    g_algo_1d.store(algo, std::memory_order_relaxed);
    return TURBOFNO_OK;
}

int turbofno_get_1d_algo(void) { return algo_1d(); }

int turbofno_set_exchange_wait_us(unsigned long long microseconds)
{
    tfno::set_cluster_wait_ticks(microseconds > (~0ull) / 100 ? ~0ull : microseconds * 100);   // 100 MHz wall clock   // 100 MHz wall clock
    return TURBOFNO_OK;
}

size_t turbofno_exchange_bytes(int compute_units) { return tfno::exchange_bytes(compute_units); }

int turbofno_exchange_attach(void* stream, void* buffer, size_t bytes)
{
    if (!buffer) return fail(TURBOFNO_ERR_INVALID_ARG, "buffer must be a non-null device pointer (turbofno_exchange_detach forgets a buffer)");
    const hipError_t e = tfno::exchange_attach((hipStream_t)stream, buffer, bytes);
    if (e == hipErrorInvalidValue)
        return fail(TURBOFNO_ERR_WORKSPACE, "exchange buffer must be 256-byte aligned and hold turbofno_exchange_bytes(0) = %zu bytes (%zu given)",
                    tfno::exchange_bytes(0), bytes);
    if (e == hipErrorStreamCaptureUnsupported)
        return fail(TURBOFNO_ERR_INVALID_ARG, "the stream is being captured: attach the exchange buffer before the capture begins");
    return hip_status(e, "exchange_attach");
}

int turbofno_exchange_detach(void* stream) { return hip_status(tfno::exchange_attach((hipStream_t)stream, nullptr, 0), "exchange_detach"); }

int turbofno_exchange_status(void* stream, unsigned* gave_up)
{
    unsigned count = 0;
    const hipError_t e = tfno::exchange_gave_up((hipStream_t)stream, &count);
    if (e == hipErrorNotReady) {                                 // nothing attached: nothing can have waited
        if (gave_up) *gave_up = 0;
        return TURBOFNO_OK;
    }
    if (int rc = hip_status(e, "exchange_status")) return rc;
    if (gave_up) *gave_up = count;
    if (count)
        return fail(TURBOFNO_ERR_EXCHANGE, "%u cluster member(s) on this stream did not get the other members' partial products in time "
                                           "and computed their share themselves since the last call: results are valid, those "
                                           "launches were slow", count);
    return TURBOFNO_OK;
}

int turbofno_query_1d_kernel(int logDY, long M, int N, int K, int compute_units, int exchange_attached)
{
    if (check_gemm_dims(M, N, K) || !length_built(logDY)) return 0;
    const long cus = compute_units > 0 ? compute_units : tfno::cu_count();
    return tfno::pick_fused_1d_kernel(logDY, M / 64, N, K, algo_1d(), false, cus, exchange_attached != 0);
}

int turbofno_query_2d_algo(int bs, int DX, int DY, int K, int N, int algo)
{
    if (bs <= 0 || K <= 0 || N <= 0 || K % 8 || N % 64) return 0;
    const int logDX = log2_exact(DX), logDY = log2_exact(DY);
    if (!length_built(logDX) || !length_built(logDY)) return 0;
    if (algo < TURBOFNO_2D_AUTO || algo > TURBOFNO_2D_ROWS_FIRST) return 0;
    if (algo == TURBOFNO_2D_WHOLE_IMAGE && !whole_image_built(DX, DY)) return 0;
    return pick_algo(bs, DX, DY, K, N, algo);
}

int turbofno_fused_fft_cgemm_ifft(int logDY, long M, int N, int K, const void* x, const void* W, void* C, void* y,
                                  float alpha_re, float alpha_im, float beta_re, float beta_im, void* stream)
{
    (void)C; (void)beta_re; (void)beta_im;
    if (!x || !W || !y) return fail(TURBOFNO_ERR_INVALID_ARG, "x, W and y must be non-null device pointers");
    if (int rc = check_gemm_dims(M, N, K)) return rc;
    if (!length_built(logDY)) return fail(TURBOFNO_ERR_UNSUPPORTED, "log2(DY)=%d: only DY in {128, 256, 512, 1024} is built", logDY);
    if (M / 64 > 0x7fffffffL) return fail(TURBOFNO_ERR_INVALID_ARG, "M/64=%ld exceeds the grid limit", M / 64);
    hipError_t e = tfno::launch_fused_fft_cgemm_ifft(logDY, M / 64, N, K, (const float2*)x, (const float2*)W, (float2*)y,
                                                     make_float2(alpha_re, alpha_im), algo_1d(), (hipStream_t)stream);
    return hip_status(e, "fused_fft_cgemm_ifft launch");
}

static int stride_common(bool inverse, int logDX, const void* in, void* out, int DY, long total, int dimX, void* stream)
{
    if (!in || !out) return fail(TURBOFNO_ERR_INVALID_ARG, "in and out must be non-null device pointers");
    if (dimX != TURBOFNO_MODES) return fail(TURBOFNO_ERR_INVALID_ARG, "dimX=%d: exactly 64 rows are retained", dimX);
    if (DY <= 0 || DY % 16) return fail(TURBOFNO_ERR_INVALID_ARG, "DY=%d must be a positive multiple of 16", DY);
    if (total <= 0 || total % DY) return fail(TURBOFNO_ERR_INVALID_ARG, "total=%ld must be a positive multiple of DY=%d", total, DY);
    if (!length_built(logDX)) return fail(TURBOFNO_ERR_UNSUPPORTED, "log2(DX)=%d: only DX in {128, 256, 512, 1024} is built", logDX);
    hipError_t e = inverse ? tfno::launch_ifft_stride(logDX, (const float2*)in, (float2*)out, DY, total / DY, (hipStream_t)stream)
                           : tfno::launch_fft_stride(logDX, (const float2*)in, (float2*)out, DY, total / DY, (hipStream_t)stream);
    return hip_status(e, inverse ? "ifft_stride launch" : "fft_stride launch");
}

int turbofno_fft_stride(int logDX, const void* in, void* out, int threadblock_bs, int DY, long total, int dimX, void* stream)
{
    (void)threadblock_bs;
    return stride_common(false, logDX, in, out, DY, total, dimX, stream);
}

int turbofno_ifft_stride(int logDX, const void* in, void* out, int threadblock_bs, int DY, long total, int dimX, void* stream)
{
    (void)threadblock_bs;
    return stride_common(true, logDX, in, out, DY, total, dimX, stream);
}

int turbofno_layer_1d(int bs, int dimX, int DY, int K, int N, const void* x, const void* W, void* y, float alpha_re,
                      float alpha_im, void* stream)
{
    if (bs <= 0 || dimX <= 0) return fail(TURBOFNO_ERR_INVALID_ARG, "bs=%d and dimX=%d must be positive", bs, dimX);
    int logDY = log2_exact(DY);
    if (logDY < 0) return fail(TURBOFNO_ERR_INVALID_ARG, "DY=%d is not a power of two", DY);
    return turbofno_fused_fft_cgemm_ifft(logDY, (long)bs * dimX * 64, N, K, x, W, nullptr, y, alpha_re, alpha_im, 0.f, 0.f, stream);
}

int turbofno_fft2d_trunc(int DX, int DY, const void* x, void* spec, long nimg, void* stream)
{
    if (!x || !spec) return fail(TURBOFNO_ERR_INVALID_ARG, "x and spec must be non-null device pointers");
    if (nimg <= 0 || nimg > 0x7fffffffL) return fail(TURBOFNO_ERR_INVALID_ARG, "nimg=%ld out of range", nimg);
    const int logDX = log2_exact(DX), logDY = log2_exact(DY);
    if (!image_length_built(logDX) || !length_built(logDY))
        return fail(TURBOFNO_ERR_UNSUPPORTED, "DX=%d, DY=%d: the stand-alone image transforms are built for DX in {128, 256} and DY in {128, 256, 512, 1024}", DX, DY);
    return hip_status(tfno::launch_fft2d_trunc(logDX, logDY, (const float2*)x, (float2*)spec, nimg, (hipStream_t)stream), "fft2d_trunc launch");
}

int turbofno_ifft2d_pad(int DX, int DY, const void* spec, void* y, long nimg, void* stream)
{
    if (!spec || !y) return fail(TURBOFNO_ERR_INVALID_ARG, "spec and y must be non-null device pointers");
    if (nimg <= 0 || nimg > 0x7fffffffL) return fail(TURBOFNO_ERR_INVALID_ARG, "nimg=%ld out of range", nimg);
    const int logDX = log2_exact(DX), logDY = log2_exact(DY);
    if (!image_length_built(logDX) || !length_built(logDY))
        return fail(TURBOFNO_ERR_UNSUPPORTED, "DX=%d, DY=%d: the stand-alone image transforms are built for DX in {128, 256} and DY in {128, 256, 512, 1024}", DX, DY);
    return hip_status(tfno::launch_ifft2d_pad(logDX, logDY, (const float2*)spec, (float2*)y, nimg, (hipStream_t)stream), "ifft2d_pad launch");
}

int turbofno_cgemm(long M, int N, int K, const void* A, const void* B, void* C, float alpha_re, float alpha_im,
                   float beta_re, float beta_im, void* stream)
{
    if (!A || !B || !C) return fail(TURBOFNO_ERR_INVALID_ARG, "A, B and C must be non-null device pointers");
    if (int rc = check_gemm_dims(M, N, K)) return rc;
    if (M >= (1L << 27)) return fail(TURBOFNO_ERR_INVALID_ARG, "M=%ld exceeds the 2^27 rows the 32-bit lane offsets cover", M);
    return hip_status(tfno::launch_cgemm_modes((const float2*)A, (const float2*)B, (float2*)C, M, N, K,
                                               make_float2(alpha_re, alpha_im), make_float2(beta_re, beta_im),
                                               (hipStream_t)stream), "cgemm launch");
}

static int stride_DY_common(bool inverse, int logDY, const void* in, void* out, long total, void* stream)
{
    if (!in || !out) return fail(TURBOFNO_ERR_INVALID_ARG, "in and out must be non-null device pointers");
    if (total <= 0) return fail(TURBOFNO_ERR_INVALID_ARG, "total=%ld must be positive", total);
    if (!length_built(logDY)) return fail(TURBOFNO_ERR_UNSUPPORTED, "log2(DY)=%d: only DY in {128, 256, 512, 1024} is built", logDY);
    hipError_t e = inverse ? tfno::launch_ifft_stride_DY(logDY, (const float2*)in, (float2*)out, total, (hipStream_t)stream)
                           : tfno::launch_fft_stride_DY(logDY, (const float2*)in, (float2*)out, total, (hipStream_t)stream);
    return hip_status(e, inverse ? "ifft_stride_DY launch" : "fft_stride_DY launch");
}

int turbofno_fft_stride_DY(int logDY, const void* in, void* out, int threadblock_bs, long total, void* stream)
{
    (void)threadblock_bs;
    return stride_DY_common(false, logDY, in, out, total, stream);
}

int turbofno_ifft_stride_DY(int logDY, const void* in, void* out, int threadblock_bs, long total, void* stream)
{
    (void)threadblock_bs;
    return stride_DY_common(true, logDY, in, out, total, stream);
}

int turbofno_fused_fft_cgemm(int logDY, long M, int N, int K, const void* x, const void* W, void* C, float alpha_re,
                             float alpha_im, float beta_re, float beta_im, void* stream)
{
    if (!x || !W || !C) return fail(TURBOFNO_ERR_INVALID_ARG, "x, W and C must be non-null device pointers");
    if (int rc = check_gemm_dims(M, N, K)) return rc;
    if (!length_built(logDY)) return fail(TURBOFNO_ERR_UNSUPPORTED, "log2(DY)=%d: only DY in {128, 256, 512, 1024} is built", logDY);
    if (M / 64 > 0x7fffffffL) return fail(TURBOFNO_ERR_INVALID_ARG, "M/64=%ld exceeds the grid limit", M / 64);
    return hip_status(tfno::launch_fused_fft_cgemm(logDY, M / 64, N, K, (const float2*)x, (const float2*)W, (float2*)C,
                                                   make_float2(alpha_re, alpha_im), make_float2(beta_re, beta_im),
                                                   (hipStream_t)stream), "fused_fft_cgemm launch");
}

int turbofno_fused_cgemm_ifft(int logDY, long M, int N, int K, const void* A, const void* W, void* C, void* y,
                              float alpha_re, float alpha_im, float beta_re, float beta_im, void* stream)
{
    (void)C; (void)beta_re; (void)beta_im;
    if (!A || !W || !y) return fail(TURBOFNO_ERR_INVALID_ARG, "A, W and y must be non-null device pointers");
    if (int rc = check_gemm_dims(M, N, K)) return rc;
    if (!length_built(logDY)) return fail(TURBOFNO_ERR_UNSUPPORTED, "log2(DY)=%d: only DY in {128, 256, 512, 1024} is built", logDY);
    if (M / 64 > 0x7fffffffL) return fail(TURBOFNO_ERR_INVALID_ARG, "M/64=%ld exceeds the grid limit", M / 64);
    return hip_status(tfno::launch_fused_cgemm_ifft(logDY, M / 64, N, K, (const float2*)A, (const float2*)W, (float2*)y,
                                                    make_float2(alpha_re, alpha_im), (hipStream_t)stream),
                      "fused_cgemm_ifft launch");
}

size_t turbofno_layer_2d_workspace_bytes(int bs, int DX, int DY, int K, int N, int algo)
{
    if (bs <= 0 || DX <= 0 || DY <= 0 || K <= 0 || N <= 0) return 0;
    if (pick_algo(bs, DX, DY, K, N, algo) == TURBOFNO_2D_WHOLE_IMAGE)
        return align256((size_t)image_parts(DX) * K * bs * 4096 * sizeof(float2)) + align256((size_t)N * bs * 4096 * sizeof(float2));
    const int kept_rows_of = pick_algo(bs, DX, DY, K, N, algo) == TURBOFNO_2D_ROWS_FIRST ? DX : DY;
    return align256((size_t)K * bs * 64 * kept_rows_of * sizeof(float2)) + align256((size_t)N * bs * 64 * kept_rows_of * sizeof(float2));
}

// Both 2D entry points: validation, choice of algorithm, the three launches. `workspace` is the caller's buffer
// (turbofno_layer_2d) or this GPU's copy of the static scratch array (turbofno_layer_2d_noalloc); `what` names it
// in error messages.
static int layer_2d_on(int bs, int DX, int DY, int K, int N, const void* x, const void* W, void* y, float alpha_re,
                       float alpha_im, void* workspace, size_t workspace_bytes, const char* what, int algo, void* stream)
{
    if (!x || !W || !y) return fail(TURBOFNO_ERR_INVALID_ARG, "x, W and y must be non-null device pointers");
    if (bs <= 0) return fail(TURBOFNO_ERR_INVALID_ARG, "bs=%d must be positive", bs);
    int logDX = log2_exact(DX), logDY = log2_exact(DY);
    if (logDX < 0 || logDY < 0) return fail(TURBOFNO_ERR_INVALID_ARG, "DX=%d, DY=%d must be powers of two", DX, DY);
    if (int rc = check_gemm_dims((long)bs * 64 * 64, N, K)) return rc;
    if ((long)K * bs > 0x7fffffffL || (long)N * bs > 0x7fffffffL)
        return fail(TURBOFNO_ERR_INVALID_ARG, "K*bs=%ld or N*bs=%ld images exceed the grid limit", (long)K * bs, (long)N * bs);
    if (!length_built(logDX) || !length_built(logDY))
        return fail(TURBOFNO_ERR_UNSUPPORTED, "DX=%d, DY=%d: only lengths in {128, 256, 512, 1024} are built", DX, DY);
    if (algo != TURBOFNO_2D_AUTO && algo != TURBOFNO_2D_THREE_KERNEL && algo != TURBOFNO_2D_WHOLE_IMAGE && algo != TURBOFNO_2D_ROWS_FIRST)
        return fail(TURBOFNO_ERR_INVALID_ARG, "unknown algo %d", algo);
    if (algo == TURBOFNO_2D_WHOLE_IMAGE && !whole_image_built(DX, DY))
        return fail(TURBOFNO_ERR_UNSUPPORTED, "DX=%d, DY=%d: the whole-image path is built for DY in {128, 256} and DX in {128, 256, 512, 1024}", DX, DY);
    const int a = pick_algo(bs, DX, DY, K, N, algo);
    const size_t need = turbofno_layer_2d_workspace_bytes(bs, DX, DY, K, N, a);
    if (!workspace || workspace_bytes < need)
        return fail(TURBOFNO_ERR_WORKSPACE, "%s of %zu bytes required, %zu available", what, need, workspace ? workspace_bytes : (size_t)0);
    if ((size_t)workspace % 256) return fail(TURBOFNO_ERR_WORKSPACE, "%s must be 256-byte aligned", what);
    hipStream_t st = (hipStream_t)stream;
    const float2 alpha = make_float2(alpha_re, alpha_im);
    char* ws = (char*)workspace;
    if (a == TURBOFNO_2D_WHOLE_IMAGE) {
        const int parts = image_parts(DX);         // DX above 256: the parts of an image are channels of the contraction
        float2* spec = (float2*)ws;
        float2* cspec = (float2*)(ws + align256((size_t)parts * K * bs * 4096 * sizeof(float2)));
        if (int rc = hip_status(tfno::launch_fft2d_trunc(logDX, logDY, (const float2*)x, spec, K * bs, st), "fft2d_trunc launch")) return rc;
        if (int rc = hip_status(tfno::launch_cgemm_modes(spec, (const float2*)W, cspec, (long)bs * 4096, N, parts * K, alpha, make_float2(0.f, 0.f), st, K), "cgemm_modes launch")) return rc;
        return hip_status(tfno::launch_ifft2d_pad(logDX, logDY, cspec, (float2*)y, N * bs, st), "ifft2d_pad launch");
    }
    if (a == TURBOFNO_2D_ROWS_FIRST) {
        float2* t1 = (float2*)ws;
        float2* t2 = (float2*)(ws + align256((size_t)K * bs * 64 * DX * sizeof(float2)));
        if (int rc = hip_status(tfno::launch_fft_rows_trunc(logDY, (const float2*)x, t1, DX, (long)K * bs, st), "fft_rows_trunc launch")) return rc;
        if (int rc = hip_status(tfno::launch_fused_fft_cgemm_ifft(logDX, (long)bs * 64, N, K, t1, (const float2*)W, t2, alpha, algo_1d(), st, /*y_is_reread=*/true), "fused_fft_cgemm_ifft launch")) return rc;
        return hip_status(tfno::launch_ifft_rows_pad(logDY, t2, (float2*)y, DX, (long)N * bs, st), "ifft_rows_pad launch");
    }
    float2* t1 = (float2*)ws;
    float2* t2 = (float2*)(ws + align256((size_t)K * bs * 64 * DY * sizeof(float2)));
    if (int rc = hip_status(tfno::launch_fft_stride(logDX, (const float2*)x, t1, DY, (long)K * bs, st), "fft_stride launch")) return rc;
    if (int rc = hip_status(tfno::launch_fused_fft_cgemm_ifft(logDY, (long)bs * 64, N, K, t1, (const float2*)W, t2, alpha, algo_1d(), st, /*y_is_reread=*/true), "fused_fft_cgemm_ifft launch")) return rc;
    return hip_status(tfno::launch_ifft_stride(logDX, t2, (float2*)y, DY, (long)N * bs, st), "ifft_stride launch");
}

int turbofno_layer_2d(int bs, int DX, int DY, int K, int N, const void* x, const void* W, void* y, float alpha_re,
                      float alpha_im, void* workspace, size_t workspace_bytes, int algo, void* stream)
{
    return layer_2d_on(bs, DX, DY, K, N, x, W, y, alpha_re, alpha_im, workspace, workspace_bytes, "workspace", algo, stream);
}

// ---- the 2D layer for callers that cannot allocate -------------------------------------------------------------
// The intermediates of the layer live in a file-scope device array instead of a caller-provided workspace. Every GPU
// holds its own copy of the array at its own address (from module load until the process ends); that address is
// resolved once per device, with that device current, and kept. Host code uses the resolved pointer only: the
// array's name is a host-side stand-in, not a device address.
static __device__ __align__(256) unsigned char scratch[TURBOFNO_NOALLOC_SCRATCH_BYTES];
static std::atomic<void*> g_scratch_ptr[64];

static int scratch_of_current_device(void* stream, void** out)
{
    int dev = 0;
    if (int rc = hip_status(hipGetDevice(&dev), "hipGetDevice")) return rc;
    // The kernels run on the stream's device and must get THAT device's copy of the array. A launch on a stream of
    // another device than the current one is refused rather than resolved behind the caller's back.
    if (stream && (hipStream_t)stream != hipStreamPerThread && (hipStream_t)stream != hipStreamLegacy) {
        int sdev = dev;
        if (int rc = hip_status(hipStreamGetDevice((hipStream_t)stream, &sdev), "hipStreamGetDevice")) return rc;
        if (sdev != dev)
            return fail(TURBOFNO_ERR_INVALID_ARG, "the stream belongs to device %d, the current device is %d: make the stream's device current", sdev, dev);
    }
    if (dev < 0 || dev >= 64) return fail(TURBOFNO_ERR_UNSUPPORTED, "device ordinal %d: the static scratch is tracked for ordinals below 64", dev);
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        if (int rc = hip_status(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return rc;
        if (!p) return fail(TURBOFNO_ERR_HIP, "hipGetSymbolAddress(scratch) returned a null address");
        g_scratch_ptr[dev].store(p, std::memory_order_release);       // a racing thread resolves the same address
    }
    *out = p;
    return TURBOFNO_OK;
}

int turbofno_layer_2d_noalloc(int bs, int DX, int DY, int K, int N, const void* x, const void* W, void* y,
                              float alpha_re, float alpha_im, int algo, void* stream)
{
    // sizes first, so that an oversized problem is refused without touching the device
    if (bs > 0 && DX > 0 && DY > 0 && K > 0 && N > 0) {
        const size_t need = turbofno_layer_2d_workspace_bytes(bs, DX, DY, K, N, algo);
        if (need > (size_t)TURBOFNO_NOALLOC_SCRATCH_BYTES)
            return fail(TURBOFNO_ERR_WORKSPACE,
                        "the layer needs %zu bytes of intermediates, the static scratch holds %zu: use turbofno_layer_2d with "
                        "a workspace, or split the batch", need, (size_t)TURBOFNO_NOALLOC_SCRATCH_BYTES);
    }
    void* ptr = nullptr;
    if (int rc = scratch_of_current_device(stream, &ptr)) return rc;
    return layer_2d_on(bs, DX, DY, K, N, x, W, y, alpha_re, alpha_im, ptr, (size_t)TURBOFNO_NOALLOC_SCRATCH_BYTES,
                       "static scratch", algo, stream);
}

}  // extern "C"
