// Whole-image 2D spectral layer (the MI355X-first path of the 2D layer): images of DX x DY with DX in {128, 256} rows
// per block - 512 and 1024 rows as two and four interleaved parts of 256 ("decimated images" below) - and rows of DY in
// {128, 256, 512, 1024}.
//
// The reference's "fully fused" 2D variant is three kernels with two HBM round trips of
// half-truncated intermediates (fusion_variants/2D_D_exp_fused_fft_cgemm_ifft/fused_trunc_2D.cu:150-172:
// X transform -> t1[K*bs][64][DY], fused Y stage, t2[N*bs][64][DY] -> X inverse). Here one 1024-thread
// block owns a whole DX x DY image, so only fully truncated 64 x 64 spectra ever leave the CU:
//
//   fft2d_trunc    image (k,b): DX row FFTs along Y (coalesced rows, 64 modes kept, held in registers),
//                  redistribution through LDS, 64 column FFTs along X (64 modes kept)
//                  -> spec[k][b][4096]                          reads 8 DX DY bytes, writes 32 KiB
//   cgemm_modes    C[n][b][m] = alpha * sum_k W[k][n] spec[k][b][m] on the fp32 matrix cores
//   ifft2d_pad     exact mirror -> y[n][b][DX][DY]              reads 32 KiB, writes 8 DX DY bytes
//
// so x is read once and y written once; padded / discarded modes are never touched in memory.
// The 4096 modes of an image are stored in "lane order": element mm*(64 LX) + q*LX + t holds mode
// (p = t + LX mm, q), LX = DX/16. That order is private to the two image kernels (producer and consumer
// lanes coincide, every access is contiguous per wavefront) and the GEMM is oblivious to it.
#include "group_fft.h"
#include "kernels.h"
#include <string>
#include <type_traits>

namespace tfno {

namespace {
constexpr int TPITCH = 66;                       // row pitch (complex) of the DX x 64 redistribution tile
constexpr int EXCH_ELEMS = 1024 * 17;            // exchange regions of all lane groups of a 1024-thread block

// Geometry of the whole-image kernels for a DX x DY image (DX rows of DY contiguous samples).
// Rows of 256: a 16-lane group owns one row (16 samples per lane). Rows of 128 ("paired"): a 16-lane group owns
// two rows, 8 samples per lane each, so that a group still covers 128 contiguous bytes per access. Rows of 512 / 1024
// ("wide"): a group of 32 / 64 lanes owns one row, 16 samples per lane, 256 / 512 contiguous bytes per access.
template <int LOGX, int LOGY> struct Geo2D {
    static constexpr int DX = 1 << LOGX, DY = 1 << LOGY;
    static constexpr bool PAIRED = LOGY == 7;
    static constexpr bool WIDE = LOGY >= 9;                   // rows of 512 / 1024: 32 / 64 lanes per row
    static constexpr int LX = DX / 16, LY = WIDE ? DY / 16 : 16;   // lanes per column / per row-pass group
    static constexpr int GY = 1024 / LY;                      // lane groups of the row pass
    static constexpr int RPP = PAIRED ? 2 * GY : GY;          // rows per pass
    static constexpr int ITY = DX / RPP;                      // row passes per image
    static constexpr int MMY = PAIRED ? 8 : 64 / LY;          // modes per lane after one row pass
    static constexpr int MMX = 64 / LX;                       // modes per lane after the column pass
    static constexpr int COLT = 64 * LX;                      // threads that take part in the column pass
    static constexpr int TILE = DX * TPITCH;
    static constexpr int LDS_MAIN = EXCH_ELEMS > TILE ? EXCH_ELEMS : TILE;   // exchange regions alias the tile
    // after them: first-pass twiddles of the rows (one table row per lane of a group) and of the columns, and for rows
    // of 512 / 1024 the powers w_LY^e, e < LY, of the second pass
    static constexpr int TWY_ELEMS = LY * kTwLdsPitch, WSM_ELEMS = WIDE ? LY : 0;
    static constexpr size_t LDS_BYTES = sizeof(float2) * (size_t)(LDS_MAIN + TWY_ELEMS + kTwLdsSize + WSM_ELEMS);
    static_assert(LOGY >= 7 && LOGY <= 10, "rows of 128 to 1024");
    static_assert(ITY >= 1 && COLT <= 1024 && GY * LY * 17 <= EXCH_ELEMS, "unsupported image shape");
    // element offset of the lane's i-th sample from its first one
    // (logr: the rows of the image lie 2^logr rows of the array apart, see the decimated images below)
    static __device__ __forceinline__ constexpr int sample_off(int i, int logr = 0)
    {
        return PAIRED ? (i & 7) * 16 + (i >> 3) * ((4 * DY) << logr) : LY * i;
    }
    // column of the redistribution tile (mode along Y) that lane t of a row group holds in slot mm
    static __device__ __forceinline__ constexpr int tile_col(int t, int mm) { return PAIRED ? (t & 7) + 8 * mm : t + LY * mm; }
};

// First row (within one pass) of lane group g. The two groups that share an LDS cycle (one half wavefront) must
// hit disjoint banks of the pitch-66 tile, i.e. sit 8 rows apart (4 rows = 16 banks).
//   rows of 256: one row per group; groups 2j, 2j+1 get rows 8 apart.
//   rows of 128: group g owns rows a and a + 4 (lanes 0-7 / 8-15 finish one each: 16 banks apart), a enumerating the
//   rows with bit 2 clear; groups 2j, 2j+1 again 8 rows apart.
//   rows of 512 / 1024: one row per group, a group is at least half a wavefront: any order.
template <bool PAIRED, bool WIDE = false> __device__ __forceinline__ int first_row_in_pass(int g)
{
    const int jh = g & 1, rest = g >> 1;
    if constexpr (WIDE) return g;
    else if constexpr (!PAIRED) return jh * 8 + (rest % 8) + (rest / 8) * 16;
    else {
        const int s = jh * 4 + (rest % 4) + (rest / 4) * 8;    // pair index, partner groups 4 apart
        return (s & 3) + 8 * (s >> 2);
    }
}

// Decimated images (LOGR > 0): an image of R DX x DY, R = 2^LOGR, too long along X for one block, is handled as R parts
// of DX x DY: part r holds the rows R j + r. Its transform along X splits exactly (one radix-R decimation in time step):
//     X[p] = sum_{r<R} w_{R DX}^(r p) * DFT_DX(part r)[p],    p < 64
// so the forward kernel transforms every part like an image of its own and multiplies its 64 x 64 modes by w^(r p); the
// sum over r is a sum over "channels" and is done by the contraction that follows (channel r K + k, weight W[k]): the
// spectrum of part r of image i is stored at index r * nfull + i for that, nfull whole images. Backward, the R parts of
// an output image are transformed from the one spectrum of the image, multiplied by conj(w^(r p)). Nothing but x, y and
// the 64 x 64 modes ever leaves a CU, as for images of one block.
//
// Numbering of the block-images (one per block iteration). Side by side: image * R + part, the parts of an image run on
// neighbouring blocks at the same time and all rows of the array are in flight together, not every R-th one; part major:
// part * nfull + image. Measured: the forward kernels are 2-9 % faster side by side everywhere; the backward kernels as
// well for four parts and for rows up to 256, but 3 % slower for two parts of rows of 512 / 1024, which keep part major.
template <int LOGR, bool PART_MAJOR> struct PartNumbering {
    static constexpr int R = 1 << LOGR;
    static __device__ __forceinline__ unsigned part(long img, int nfull)
    {
        if constexpr (LOGR == 0) return 0;
        else if constexpr (PART_MAJOR) return (unsigned)img / (unsigned)nfull;
        else return (unsigned)img & (R - 1);
    }
    static __device__ __forceinline__ long image(long img, int nfull)
    {
        if constexpr (LOGR == 0) return img;
        else if constexpr (PART_MAJOR) return (unsigned)img % (unsigned)nfull;
        else return img >> LOGR;
    }
};
// first row in the array of block-image img: row `part` of image `image`, whose rows lie R rows apart
template <int LOGX, int LOGR, bool PART_MAJOR> __device__ __forceinline__ long first_array_row(long img, int nfull)
{
    using P = PartNumbering<LOGR, PART_MAJOR>;
    return (P::image(img, nfull) << (LOGX + LOGR)) + P::part(img, nfull);
}
constexpr int kDecimationTwiddles = 64 * 4;      // complex elements: R <= 4 parts
template <int LOGD> __device__ __forceinline__ void fill_decimation_twiddles(float2* tab, int tid, int nthreads)
{
    for (int e = tid; e < kDecimationTwiddles; e += nthreads)
        tab[e] = kTwiddle1024[(((e >> 6) * (e & 63)) << (10 - LOGD)) & 1023];
}
}  // namespace

// Forward image kernel: truncated 2D transform of one DX x DY image per block iteration.
// 1024 threads = 16 waves per CU (4 per SIMD: the arithmetic is issue bound, so full occupancy matters more
// than registers). A block is persistent over images (img = blockIdx.x, += gridDim.x). Pass 1 transforms the
// rows (along Y) with LY-lane groups and keeps the 64 retained modes of every row in registers; a pitch-66
// LDS tile redistributes them; pass 2 transforms the 64 columns (along X) with LX-lane groups.
// Each group keeps ONE row in flight: the loads of its next row are issued as soon as the first radix-4
// stage has consumed the row registers, so they travel while the rest of the transform runs, across the
// column pass and across image boundaries. Inter-pass twiddles live in LDS to stay within 128 VGPRs.
// nimg counts block-images: the 2^LOGR parts of each of the nfull whole images (nimg = nfull when LOGR = 0).
template <int LOGX, int LOGY, int LOGR>
__global__ __launch_bounds__(1024) void fft2d_trunc_kernel(const float2* __restrict__ x, float2* __restrict__ spec,
                                                           int nimg, int nfull)
{
    using G = Geo2D<LOGX, LOGY>;
    constexpr int DY = G::DY, LX = G::LX, LY = G::LY, ITY = G::ITY, MMY = G::MMY, MMX = G::MMX;
    extern __shared__ float2 lds[];
    const int tid = threadIdx.x;
    const int gy = tid / LY, ty = tid % LY;            // row pass: group and lane
    const int gx = tid / LX, tx = tid % LX;            // column pass: group (= column q) and lane
    float2* exch_y = lds + gy * (LY * 17);
    float2* exch_x = lds + gx * (LX * 17);
    float2* twtab_y = lds + G::LDS_MAIN;               // after the exchange regions / tile
    float2* twtab_x = twtab_y + G::TWY_ELEMS;
    float2* wsm = twtab_x + kTwLdsSize;
    float2* twsub = wsm + G::WSM_ELEMS;                // decimated images: w^(r p) of the long axis, r < R, p < 64
    fill_lds_twiddles<LOGY, LY>(twtab_y, tid, 1024);
    fill_lds_twiddles<LOGX>(twtab_x, tid, 1024);
    if (G::WIDE && tid < LY) wsm[tid] = kTwiddle1024[tid * (1024 / LY)];
    const float2* twrow_y = twtab_y + ty * kTwLdsPitch;
    const float2* twrow_x = twtab_x + tx * kTwLdsPitch;
    if constexpr (LOGR > 0) fill_decimation_twiddles<LOGX + LOGR>(twsub, tid, 1024);
    __syncthreads();

    const int row0 = first_row_in_pass<G::PAIRED, G::WIDE>(gy);
    // row the lane finishes after the exchange, and its first mode (paired rows: lanes 8-15 take the second row)
    const int trow = G::PAIRED ? row0 + 4 * (ty >> 3) : row0;
    // scalar base + 32-bit lane offset keeps the load addresses out of the vector registers
    const unsigned lane_off = (unsigned)(((row0 * DY) << LOGR) + ty);
    // x is streamed exactly once: non-temporal loads keep it from evicting the 64x64 spectra, which the
    // next kernel re-reads, out of L2 / Infinity Cache
    auto issue = [&](cpx (&dst)[16], long array_row, int it, unsigned off) {
        const float2* base = x + (array_row + ((G::RPP * it) << LOGR)) * (long)DY;
#pragma unroll
        for (int i = 0; i < 16; ++i) dst[i] = load_streaming(&base[off + (unsigned)G::sample_off(i, LOGR)]);
    };

    long img = blockIdx.x;
    long img_row = first_array_row<LOGX, LOGR, false>(img < nimg ? img : 0, nfull);
    cpx v[16];
    if (img < nimg) issue(v, img_row, 0, lane_off);
    for (; img < nimg; img += gridDim.x) {
        // look-ahead target: the next image's first rows; after the last image every lane group re-reads the
        // same row (row 0 of image 0, cache resident) so the loop stays branch free at no HBM cost
        const bool more = img + gridDim.x < nimg;
        const long pre_row = first_array_row<LOGX, LOGR, false>(more ? img + gridDim.x : 0, nfull);
        const unsigned pre_off = more ? lane_off : (unsigned)ty;
        // pass 1: rows (along Y). T[it][mm] = mode tq + 16 mm (paired rows: tq + 8 mm) of row trow + RPP it
        cpx T[ITY][MMY];
#pragma unroll
        for (int it = 0; it < ITY; ++it) {
            if constexpr (!G::PAIRED) {
                cpx bb[16], gg[16];
                fft16_stage1<-1>(v, bb);
                // v is dead after the first radix-4 stage: its registers become the landing zone of the next row;
                // the last pass already fetches the next image's first row
                if (it + 1 < ITY) issue(v, img_row, it + 1, lane_off);
                else issue(v, pre_row, 0, pre_off);
                fwd_pass1_lds_finish(bb, twrow_y, gg);
                if constexpr (G::WIDE) wide_rows_forward_finish<LY>(gg, exch_y, wsm, ty, T[it]);
                else group_forward_finish<8>(gg, exch_y, ty, T[it]);
            } else {
                cpx gg[16], b8[8];
                {
                    cpx a8[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) { a8[i] = v[i]; b8[i] = v[8 + i]; }
                    fft8<-1>(a8);
                    fft8<-1>(b8);
#pragma unroll
                    for (int r = 0; r < 8; ++r) gg[r] = a8[r];
                }
                if (it + 1 < ITY) issue(v, img_row, it + 1, lane_off);
                else issue(v, pre_row, 0, pre_off);
                gg[8] = b8[0];
#pragma unroll
                for (int r = 1; r < 8; ++r) {
                    const cpx w = twrow_y[r];
                    gg[r] = cmul(gg[r], w);
                    gg[8 + r] = cmul(b8[r], w);
                }
                rows128_forward_finish(gg, exch_y, ty, T[it]);
            }
        }
        __syncthreads();
#pragma unroll
        for (int it = 0; it < ITY; ++it)
#pragma unroll
            for (int mm = 0; mm < MMY; ++mm)
                lds[(trow + G::RPP * it) * TPITCH + G::tile_col(ty, mm)] = T[it][mm];
        __syncthreads();
        // pass 2: columns (along X); group gx owns column q = gx, lane tx holds rows tx + LX i
        cpx c[16];
        if (tid < G::COLT) {
#pragma unroll
            for (int i = 0; i < 16; ++i) c[i] = lds[(tx + LX * i) * TPITCH + gx];
        }
        __syncthreads();
        if (tid < G::COLT) {
            cpx gg[16], z[MMX];
            fwd_pass1_lds(c, twrow_x, gg);
            group_forward_finish<LOGX>(gg, exch_x, tx, z);
            if constexpr (LOGR > 0) {
                // part r of a decimated image: its modes enter the sum over the parts with w^(r p) of the long axis
                const int r = (int)PartNumbering<LOGR, false>::part(img, nfull);
                if (r != 0) {
#pragma unroll
                    for (int mm = 0; mm < MMX; ++mm) z[mm] = cmul(z[mm], twsub[r * 64 + tx + LX * mm]);
                }
            }
            // lane order of the retained modes: element mm*COLT + q*LX + tx  <->  mode (p = tx + LX mm, q).
            // Written through as it is produced, so the end-of-kernel cache write-back has nothing left to flush
            // (decimated images: the spectrum of part r of image i is channel r of the contraction, index r * nfull + i)
            float2* dst = spec + (PartNumbering<LOGR, false>::part(img, nfull) * (long)nfull + PartNumbering<LOGR, false>::image(img, nfull)) * 4096;
#pragma unroll
            for (int mm = 0; mm < MMX; ++mm) store_streaming(dst + tid + G::COLT * mm, z[mm]);
        }
        img_row = pre_row;
    }
}

// Backward image kernel, mirror of the forward one: persistent blocks, 16 waves per CU, twiddles in LDS.
// The 32 KiB spectrum of the next image is fetched (a few registers per lane) while the current image's rows
// are being transformed and stored, so a CU never waits for its input between images.
//
// SHARE: the XCDs of this GPU do not store at the same rate. Workgroup b of a grid runs on XCD b mod 8, and the blocks on
// the odd XCDs need about a fifth longer per image than those on the even ones (21.3 against 17.5 us at 256 x 256, in
// every launch on every box measured; a store-only probe gives the same picture), so with the same number of images per
// block the even half of the chip idles for the last sixth of the kernel. Here blocks 2p and 2p + 1 share the images
// p, p + P, p + 2P, ... (P pairs) unevenly: of the J * ITY row passes of the pair's J images the even block takes a share
// of even_share / kEvenShareDen, in whole images plus the first row passes of one image that the two blocks split
// (each takes it last; both run its column pass). 1024 images of 256 x 256: the even block transforms 4 1/4 images, the odd one 3 3/4: 101.6 -> 96.5 us.
// Which row goes to which block does not change any value: the output is bit-identical to the equal split.
// (even_share / kEvenShareDen, see kernels.h; measured here: 17/32 and 18/32 level, -5.3 us per layer, 19/32 -3 us)

template <int LOGX, int LOGY, bool SHARE, int LOGR>
__global__ __launch_bounds__(1024) void ifft2d_pad_kernel(const float2* __restrict__ spec, float2* __restrict__ y,
                                                          int nimg, int even_share, int nfull)
{
    using G = Geo2D<LOGX, LOGY>;
    constexpr int DY = G::DY, LX = G::LX, LY = G::LY, ITY = G::ITY, MMY = G::MMY, MMX = G::MMX;
    extern __shared__ float2 lds[];
    const int tid = threadIdx.x;
    const int gy = tid / LY, ty = tid % LY;
    const int gx = tid / LX, tx = tid % LX;
    float2* exch_y = lds + gy * (LY * 17);
    float2* exch_x = lds + gx * (LX * 17);
    float2* twtab_y = lds + G::LDS_MAIN;
    float2* twtab_x = twtab_y + G::TWY_ELEMS;
    float2* wsm = twtab_x + kTwLdsSize;
    float2* twsub = wsm + G::WSM_ELEMS;
    fill_lds_twiddles<LOGY, LY>(twtab_y, tid, 1024);
    fill_lds_twiddles<LOGX>(twtab_x, tid, 1024);
    if (G::WIDE && tid < LY) wsm[tid] = kTwiddle1024[tid * (1024 / LY)];
    const float2* twrow_y = twtab_y + ty * kTwLdsPitch;
    const float2* twrow_x = twtab_x + tx * kTwLdsPitch;
    if constexpr (LOGR > 0) fill_decimation_twiddles<LOGX + LOGR>(twsub, tid, 1024);
    __syncthreads();

    const int row0 = first_row_in_pass<G::PAIRED, G::WIDE>(gy);
    const int trow = G::PAIRED ? row0 + 4 * (ty >> 3) : row0;      // row whose modes the lane takes from the tile
    const unsigned lane_off = (unsigned)(((row0 * DY) << LOGR) + ty);
    const bool col_thread = tid < G::COLT;
    // part r of a decimated image is transformed from the spectrum of the whole image
    constexpr bool PART_MAJOR = LOGR == 1 && LOGY >= 9;
    using Parts = PartNumbering<LOGR, PART_MAJOR>;
    auto spectrum_of = [&](long img) { return spec + Parts::image(img, nfull) * 4096; };

    // The block transforms `count` images, image_at(k) for k < count; of its last one, if `split`, only the row passes
    // [pass0, pass1). Without SHARE: every block the images blockIdx.x, + gridDim.x, ... in full.
    long first = blockIdx.x, step = gridDim.x, last = 0;
    int count = (int)((nimg - first + step - 1) / step), pass0 = 0, pass1 = ITY;
    bool split = false;
    if constexpr (SHARE) {
        const int pairs = gridDim.x / 2, pr = blockIdx.x >> 1, odd = blockIdx.x & 1;     // the host launches an even grid
        const int J = (nimg - pr + pairs - 1) / pairs;                                    // images of this pair
        const int even_passes = (J * ITY * even_share + kEvenShareDen / 2) / kEvenShareDen;
        const int whole = even_passes / ITY, rest = even_passes % ITY;                    // of the even block
        step = pairs;
        split = rest != 0;
        last = pr + (long)pairs * whole;                    // the image the pair splits: the last one of either block
        if (!odd) {
            first = pr;                                     // images 0 .. whole - 1 of the pair, then the first `rest` passes
            count = whole + (split ? 1 : 0);
            pass1 = rest;
        } else {
            first = pr + (long)pairs * (whole + (split ? 1 : 0));   // the pair's remaining whole images, then the other passes
            count = J - whole;
            pass0 = rest;
        }
    }
    auto image_at = [&](int k) -> long { return (SHARE && split && k == count - 1) ? last : first + step * k; };

    cpx c[MMX];
    if (count > 0 && col_thread) {
        const float2* src = spectrum_of(image_at(0));
#pragma unroll
        for (int mm = 0; mm < MMX; ++mm) c[mm] = src[tid + G::COLT * mm];
    }
    for (int k = 0; k < count; ++k) {
        const long img = image_at(k);
        const long pre = k + 1 < count ? image_at(k + 1) : img;
        const bool partial = SHARE && split && k == count - 1;
        const int it0 = partial ? pass0 : 0, it1 = partial ? pass1 : ITY;
        // pass 1: columns (p -> x) of column q = gx
        cpx u[16];
        if constexpr (LOGR > 0) {
            const int r = (int)Parts::part(img, nfull);
            if (r != 0 && col_thread) {
#pragma unroll
                for (int mm = 0; mm < MMX; ++mm) c[mm] = cmulc(c[mm], twsub[r * 64 + tx + LX * mm]);
            }
        }
        if (col_thread) group_backward_lds<LOGX>(c, twrow_x, exch_x, tx, u);
        // the exchange regions alias the tile: every wave must be done with them before the tile is written
        __syncthreads();
        if (col_thread) {
#pragma unroll
            for (int i = 0; i < 16; ++i) lds[(tx + LX * i) * TPITCH + gx] = u[i];
            // next image's spectrum (for the last image: a harmless re-read of its own 32 KiB)
            const float2* src = spectrum_of(pre);
#pragma unroll
            for (int mm = 0; mm < MMX; ++mm) c[mm] = src[tid + G::COLT * mm];
        }
        __syncthreads();
        cpx cc[ITY][MMY];
#pragma unroll
        for (int it = 0; it < ITY; ++it)
#pragma unroll
            for (int mm = 0; mm < MMY; ++mm)
                cc[it][mm] = lds[(trow + G::RPP * it) * TPITCH + G::tile_col(ty, mm)];
        __syncthreads();
        // pass 2: rows (q -> y), coalesced row stores.
        // y is written once and not re-read by this layer: non-temporal stores stop half a gigabyte of
        // dirty lines from lingering in the Infinity Cache and being written back under the next kernel's reads
#pragma unroll
        for (int it = 0; it < ITY; ++it) {
            if (SHARE && (it < it0 || it >= it1)) continue;       // uniform: row passes of the split image left to the partner
            cpx yv[16];
            if constexpr (G::PAIRED) rows128_backward(cc[it], twrow_y, exch_y, ty, yv);
            else if constexpr (G::WIDE) wide_rows_backward<LY>(cc[it], twrow_y, wsm, exch_y, ty, yv);
            else group_backward_lds<8>(cc[it], twrow_y, exch_y, ty, yv);
            // uniform base + lane offset + immediates
            float2* dst = y + (first_array_row<LOGX, LOGR, PART_MAJOR>(img, nfull) + ((G::RPP * it) << LOGR)) * (long)DY;
#pragma unroll
            for (int i = 0; i < 16; ++i) store_streaming(dst + lane_off + G::sample_off(i, LOGR), yv[i]);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Mode-space complex GEMM on the fp32 matrix cores.
//   C[n][m] = alpha * sum_k W[k + n*K] * A[k][m] (+ beta C),   A: [K][Mtot], C: [N][Mtot]  (m contiguous)
// Same contraction as the reference's cgemm / the GEMM phase of its fused kernel
// (fusion_variants/1D_A_exp_fft+cgemm+ifft/cgemm.cuh:4-205, operand layout lda=M, ldb=K, ldc=M), with three real
// products per complex one instead of four:
//   P1 = c (a + b),  P2 = (d - c) a,  P3 = (c + d) b   =>   re = P1 - P3,  im = P1 + P2      (alpha W = c + i d, A = a + i b)
// i.e. three v_mfma_f32_16x16x4_f32 per 16 n x 16 m x 4 k: 25 % less matrix work than the real-expanded product, and
// the matrix work is the part of this kernel that nothing overlaps with (all waves of the grid load, multiply and
// store in step). Rows of a tile are 16 output channels n, columns 16 consecutive m, contraction 4 channels.
// A block is 16 waves; wave w owns the 16-m strip w and the whole 64-channel n tile, so every element of A is loaded
// exactly once: the strip of a chunk sits in NG float2 registers per lane, all loads in flight while the W tile is
// built. The n tiles are the outer loop, so each is stored as soon as it is complete and its stores drain under the
// matrix work of the next ones.
//   NG    = channel groups of four per chunk that can hold data (4, 8, 12, 16 for K <= 16, 32, 48, 64): a template
//           parameter so that the loops stay unrolled and no loads or matrix work are spent on zero padding;
//   Kw    = period of W along the contraction: channel k is weighted with W[k mod Kw + n Kw] (Kw = K: the plain product;
//           Kw = K / R: the R parts of decimated images, see above, share the weights of their image's channel);
//   MULTI = K > 64: chunks of 4 NG = 32 channels with the twelve accumulator tiles of a wave kept across them
//           (125 registers; 64-channel chunks would spill); otherwise one chunk and transient accumulators.
// ---------------------------------------------------------------------------------------------
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int GEMM_KC = 64;         // channels per LDS-resident W chunk
constexpr int GEMM_THREADS = 1024;  // 16 waves x 16 m
constexpr int GEMM_MBLOCK = 256;    // m per block

// W'' tile in LDS: three planes (c, d - c, c + d) of floats at index (k / 4) * kW3Group + (k % 4) * kW3Row + n.
// An operand fetch (64 lanes: 4 k x 16 n) reads 16 consecutive floats of four rows 80 apart: one bank each. The
// build's lanes run along k, the contiguous direction of W: a group stride of 1 (mod 64 banks) puts the 64 lanes of a
// store on 64 different banks as well.
constexpr int kW3Row = 80, kW3Group = 4 * kW3Row + 1, kW3Plane = (GEMM_KC / 4) * kW3Group;

template <int NG, bool MULTI>
__global__ __launch_bounds__(GEMM_THREADS) void cgemm_modes3m_kernel(const float2* __restrict__ A,
                                                                     const float2* __restrict__ W, float2* __restrict__ C,
                                                                     long Mtot, int N, int K, float2 alpha, float2 beta,
                                                                     int Kw)
{
    extern __shared__ float sW[];                     // 3 * kW3Plane floats
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, col = lane & 15, kq = lane >> 4;
    const int n0 = blockIdx.y * 64;
    const unsigned lane_off = (unsigned)(kq * Mtot) + (unsigned)(wave * 16 + col);
    // XCD j takes the j-th eighth of the column blocks: with every eighth block (2 KiB of each of the K + N rows, which
    // lie Mtot * 8 bytes apart) an XCD keeps to one part of the memory system; 4-10 % faster once the operands exceed the
    // Infinity Cache (bs = 128), no change below
    const unsigned mb = (unsigned)xcd_contiguous(blockIdx.x, gridDim.x);
    const float2* blk = A + (long)mb * GEMM_MBLOCK;
    const bool active = (long)mb * GEMM_MBLOCK + wave * 16 < Mtot;   // Mtot is a multiple of 16, not of 256
    float2* cblk = C + (long)mb * GEMM_MBLOCK;
    const bool has_beta = beta.x != 0.f || beta.y != 0.f;

    floatx4 p1[4], p2[4], p3[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) p1[t] = p2[t] = p3[t] = floatx4{ 0.f, 0.f, 0.f, 0.f };

    // one chunk of up to 64 channels, or (MULTI) chunks of 4 NG = 32 channels with the accumulators kept across them
    constexpr int KCH = MULTI ? 4 * NG : GEMM_KC;
    for (int kc = 0; kc < (MULTI ? K : 1); kc += KCH) {
        const int kn = (K - kc) < KCH ? (K - kc) : KCH;           // multiple of 8 (caller contract)
        const bool last = !MULTI || kc + KCH >= K;
        // the wave's whole A strip of this chunk: lane (kq, col) holds channels kc + 4 g + kq, g < NG
        // (with one chunk the loads are issued before the tile build and overlap it; with several, the accumulators
        // of all tiles stay live and the strip is loaded after the build to stay inside 128 registers)
        float2 bv[NG];
        if constexpr (!MULTI) {
#pragma unroll
            for (int g = 0; g < NG; ++g)
                bv[g] = (active && 4 * g < kn) ? (blk + (long)(kc + 4 * g) * Mtot)[lane_off] : make_float2(0.f, 0.f);
        }
        if constexpr (MULTI) __syncthreads();         // the previous chunk's tile is no longer read
        // W'' tile: lanes run along k, the contiguous direction of W[k + n*K]. With a single chunk only the first
        // BUILDERS threads build it: the waves of a block start one after the other over several microseconds, and the
        // block can only go on when the last of them has passed the barrier below - which should then find nothing left
        // to do there (its own part of the tile would add a round trip to L2 after its late start)
        constexpr int BUILDERS = MULTI ? GEMM_THREADS : GEMM_THREADS / 2;
        constexpr int WPT = KCH * 64 / BUILDERS;
        if (MULTI || tid < BUILDERS) {
            float2 wv[WPT];
#pragma unroll
            for (int u = 0; u < WPT; ++u) {
                const int idx = tid + u * BUILDERS;
                const int k = idx % KCH, n = idx / KCH;
                wv[u] = (k < kn) ? W[(kc + k) % Kw + (long)(n0 + n) * Kw] : make_float2(0.f, 0.f);
            }
#pragma unroll
            for (int u = 0; u < WPT; ++u) {
                const int idx = tid + u * BUILDERS;
                const int k = idx % KCH, n = idx / KCH;
                const float c = wv[u].x * alpha.x - wv[u].y * alpha.y, d = wv[u].x * alpha.y + wv[u].y * alpha.x;
                float* dstw = &sW[(k >> 2) * kW3Group + (k & 3) * kW3Row + n];
                dstw[0] = c;
                dstw[kW3Plane] = d - c;
                dstw[2 * kW3Plane] = c + d;
            }
        }
        if constexpr (MULTI) {
#pragma unroll
            for (int g = 0; g < NG; ++g)
                bv[g] = (active && 4 * g < kn) ? (blk + (long)(kc + 4 * g) * Mtot)[lane_off] : make_float2(0.f, 0.f);
        }
        __syncthreads();
        if (!active) continue;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if constexpr (!MULTI) p1[t] = p2[t] = p3[t] = floatx4{ 0.f, 0.f, 0.f, 0.f };
            const float* wrow = &sW[kq * kW3Row + t * 16 + col];
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                const float* w = wrow + g * kW3Group;
                p1[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[0], bv[g].x + bv[g].y, p1[t], 0, 0, 0);
                p2[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[kW3Plane], bv[g].x, p2[t], 0, 0, 0);
                p3[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[2 * kW3Plane], bv[g].y, p3[t], 0, 0, 0);
            }
            if (last) {
                // D[row = 4 kq + v][col]: output channel n0 + 16 t + 4 kq + v, column m = wave * 16 + col
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    float2* p = cblk + (long)(n0 + 16 * t + 4 * kq + v) * Mtot + (wave * 16 + col);
                    float2 r = make_float2(p1[t][v] - p3[t][v], p1[t][v] + p2[t][v]);
                    if (has_beta) r = cadd(r, cmul(*p, beta));      // C = alpha A W + beta C (variants A, B)
                    *p = r;
                }
            }
        }
    }
}

// K <= 64 and several column blocks per CU: persistent. A block builds the W'' tile once and walks column blocks (XCD j the
// j-th eighth of them, in order). There is no barrier inside the walk, so the waves of a CU drift apart, and the loads of
// one, the matrix work of another and the stores of a third overlap; the strip of the next column block is requested
// before the matrix work on the current one starts. C = alpha A W only (beta = 0).
template <int NG>
__global__ __launch_bounds__(GEMM_THREADS) void cgemm_modes3m_persistent_kernel(const float2* __restrict__ A,
                                                                                const float2* __restrict__ W,
                                                                                float2* __restrict__ C, long Mtot, int N, int K,
                                                                                float2 alpha, long nblocks, int Kw)
{
    extern __shared__ float sW[];                     // 3 * kW3Plane floats
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, col = lane & 15, kq = lane >> 4;
    const int n0 = blockIdx.y * 64;
    const unsigned lane_off = (unsigned)(kq * Mtot) + (unsigned)(wave * 16 + col);
    const bool eighths = (gridDim.x & 7) == 0 && (nblocks & 7) == 0;
    auto block_of = [&](long v) { return eighths ? (v & 7) * (nblocks >> 3) + (v >> 3) : v; };
    auto fetch = [&](float2 (&dst)[NG], long mb) {
        const bool active = mb * GEMM_MBLOCK + wave * 16 < Mtot;      // Mtot is a multiple of 16, not of 256
        const float2* blk = A + mb * GEMM_MBLOCK;
#pragma unroll
        for (int g = 0; g < NG; ++g) dst[g] = (active && 4 * g < K) ? (blk + (long)(4 * g) * Mtot)[lane_off] : make_float2(0.f, 0.f);
    };
    long v = blockIdx.x;                              // the grid is no larger than the number of column blocks
    float2 bv[NG];
    fetch(bv, block_of(v));
    {
        constexpr int WPT = GEMM_KC * 64 / GEMM_THREADS;
        float2 wv[WPT];
#pragma unroll
        for (int u = 0; u < WPT; ++u) {
            const int idx = tid + u * GEMM_THREADS;
            const int k = idx % GEMM_KC, n = idx / GEMM_KC;
            wv[u] = (k < K) ? W[k % Kw + (long)(n0 + n) * Kw] : make_float2(0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < WPT; ++u) {
            const int idx = tid + u * GEMM_THREADS;
            const int k = idx % GEMM_KC, n = idx / GEMM_KC;
            const float c = wv[u].x * alpha.x - wv[u].y * alpha.y, d = wv[u].x * alpha.y + wv[u].y * alpha.x;
            float* dstw = &sW[(k >> 2) * kW3Group + (k & 3) * kW3Row + n];
            dstw[0] = c;
            dstw[kW3Plane] = d - c;
            dstw[2 * kW3Plane] = c + d;
        }
    }
    __syncthreads();
    for (; v < nblocks; v += gridDim.x) {
        asm volatile("" ::: "memory");                // keeps the operand fetches from the W'' tile inside the loop (192 registers otherwise)
        const long mb = block_of(v);
        const bool more = v + gridDim.x < nblocks;
        const long nb = more ? block_of(v + gridDim.x) : mb;
        const bool next_active = more && nb * GEMM_MBLOCK + wave * 16 < Mtot;
        const float2* nblk = A + nb * GEMM_MBLOCK;
        const bool active = mb * GEMM_MBLOCK + wave * 16 < Mtot;
        float2* cblk = C + mb * GEMM_MBLOCK;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            floatx4 p1 = floatx4{ 0.f, 0.f, 0.f, 0.f }, p2 = p1, p3 = p1;
            const float* wrow = &sW[kq * kW3Row + t * 16 + col];
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                const float* w = wrow + g * kW3Group;
                p1 = __builtin_amdgcn_mfma_f32_16x16x4f32(w[0], bv[g].x + bv[g].y, p1, 0, 0, 0);
                p2 = __builtin_amdgcn_mfma_f32_16x16x4f32(w[kW3Plane], bv[g].x, p2, 0, 0, 0);
                p3 = __builtin_amdgcn_mfma_f32_16x16x4f32(w[2 * kW3Plane], bv[g].y, p3, 0, 0, 0);
                // the last n tile has used this group of the strip: its registers take the next column block's
                if (t == 3 && more) bv[g] = (next_active && 4 * g < K) ? (nblk + (long)(4 * g) * Mtot)[lane_off] : make_float2(0.f, 0.f);
            }
            if (active) {
#pragma unroll
                for (int vv = 0; vv < 4; ++vv) {
                    float2* p = cblk + (long)(n0 + 16 * t + 4 * kq + vv) * Mtot + (wave * 16 + col);
                    *p = make_float2(p1[vv] - p3[vv], p1[vv] + p2[vv]);
                }
            }
        }
    }
}

// 64 < K <= 128, beta = 0: persistent as well. The W'' tile of ALL channels (three planes of 32 channel groups, 123 KiB:
// one block per CU) is built once; a column block is multiplied in chunks of 32 channels with the accumulators of the
// four n tiles kept, the strip registers of a chunk take the next chunk (or the first chunk of the next column block) as
// soon as the last n tile has used them, and nothing inside the walk waits at a barrier.
constexpr int GEMM_KMAX = 128;
constexpr int kW3WidePlane = (GEMM_KMAX / 4) * kW3Group;
__global__ __launch_bounds__(GEMM_THREADS) void cgemm_modes3m_persistent_wide_kernel(const float2* __restrict__ A,
                                                                                     const float2* __restrict__ W,
                                                                                     float2* __restrict__ C, long Mtot, int N, int K,
                                                                                     float2 alpha, long nblocks, int Kw)
{
    extern __shared__ float sW[];                     // 3 * kW3WidePlane floats
    constexpr int NG = 8;                             // channel groups per chunk
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, col = lane & 15, kq = lane >> 4;
    const int n0 = blockIdx.y * 64;
    const unsigned lane_off = (unsigned)(kq * Mtot) + (unsigned)(wave * 16 + col);
    const bool eighths = (gridDim.x & 7) == 0 && (nblocks & 7) == 0;
    auto block_of = [&](long v) { return eighths ? (v & 7) * (nblocks >> 3) + (v >> 3) : v; };
    const int nchunks = (K + 4 * NG - 1) / (4 * NG);
    // strip of chunk c of column block mb: lane (kq, col) holds channels 32 c + 4 g + kq
    auto strip_elem = [&](long mb, int c, int g) {
        const int k = 4 * NG * c + 4 * g;
        const bool ok = mb * GEMM_MBLOCK + wave * 16 < Mtot && k < K;         // Mtot is a multiple of 16, not of 256
        return ok ? (A + mb * GEMM_MBLOCK + (long)k * Mtot)[lane_off] : make_float2(0.f, 0.f);
    };
    long v = blockIdx.x;                              // the grid is no larger than the number of column blocks
    float2 bv[NG];
#pragma unroll
    for (int g = 0; g < NG; ++g) bv[g] = strip_elem(block_of(v), 0, g);
    for (int idx = tid; idx < GEMM_KMAX * 64; idx += GEMM_THREADS) {
        const int k = idx % GEMM_KMAX, n = idx / GEMM_KMAX;
        const float2 w = (k < K) ? W[k % Kw + (long)(n0 + n) * Kw] : make_float2(0.f, 0.f);
        const float c = w.x * alpha.x - w.y * alpha.y, d = w.x * alpha.y + w.y * alpha.x;
        float* dstw = &sW[(k >> 2) * kW3Group + (k & 3) * kW3Row + n];
        dstw[0] = c;
        dstw[kW3WidePlane] = d - c;
        dstw[2 * kW3WidePlane] = c + d;
    }
    __syncthreads();
    for (; v < nblocks; v += gridDim.x) {
        asm volatile("" ::: "memory");                // keeps the operand fetches from the W'' tile inside the loop
        const long mb = block_of(v);
        const bool more = v + gridDim.x < nblocks;
        const long nb = more ? block_of(v + gridDim.x) : mb;
        floatx4 p1[4], p2[4], p3[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) p1[t] = p2[t] = p3[t] = floatx4{ 0.f, 0.f, 0.f, 0.f };
        for (int c = 0; c < nchunks; ++c) {
            const bool last = c + 1 == nchunks;
            const bool refill = !last || more;
            const long fb = last ? nb : mb;           // where the strip registers are refilled from
            const int fc = last ? 0 : c + 1;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const float* wrow = &sW[(c * NG) * kW3Group + kq * kW3Row + t * 16 + col];
#pragma unroll
                for (int g = 0; g < NG; ++g) {
                    const float* w = wrow + g * kW3Group;
                    p1[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[0], bv[g].x + bv[g].y, p1[t], 0, 0, 0);
                    p2[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[kW3WidePlane], bv[g].x, p2[t], 0, 0, 0);
                    p3[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[2 * kW3WidePlane], bv[g].y, p3[t], 0, 0, 0);
                    if (t == 3 && refill) bv[g] = strip_elem(fb, fc, g);
                }
            }
        }
        if (mb * GEMM_MBLOCK + wave * 16 < Mtot) {
            float2* cblk = C + mb * GEMM_MBLOCK;
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int vv = 0; vv < 4; ++vv)
                    cblk[(long)(n0 + 16 * t + 4 * kq + vv) * Mtot + (wave * 16 + col)] =
                        make_float2(p1[t][vv] - p3[t][vv], p1[t][vv] + p2[t][vv]);
        }
    }
}

int cu_count()
{
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    int v = cached[dev & 63].load(std::memory_order_relaxed);
    if (v > 0) return v;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
    cached[dev & 63].store(v, std::memory_order_relaxed);
    return v;
}

int even_share_parts()
{
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return kEvenShareDen / 2;
    int v = cached[dev & 63].load(std::memory_order_relaxed);
    if (v > 0) return v;
    hipDeviceProp_t prop;
    v = kEvenShareDen / 2;
    if (hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount == 256 &&
        std::string(prop.gcnArchName).rfind("gfx950", 0) == 0)
        v = 17;
    cached[dev & 63].store(v, std::memory_order_relaxed);
    return v;
}

template <int LOGX, int LOGY, int LOGR>
static hipError_t launch_image_kernel(bool inverse, const float2* in, float2* out, int nfull, hipStream_t stream)
{
    using G = Geo2D<LOGX, LOGY>;
    if (nfull <= 0 || nfull > (0x7fffffff >> LOGR)) return hipErrorInvalidValue;
    const int nimg = nfull << LOGR;                    // images of one block each: the 2^LOGR parts of every image
    const size_t lds_bytes = G::LDS_BYTES + (LOGR > 0 ? sizeof(float2) * kDecimationTwiddles : 0);
    // persistent blocks: at most as many as fit at once (LDS allows one or two 1024-thread blocks per CU,
    // the thread count exactly one)
    const int blocks = nimg < cu_count() ? nimg : cu_count();
    // uneven shares between the blocks of a pair: a full grid (one block per CU, so that block parity is XCD parity), at
    // least two images per block (128 x 128 images are a single row pass each and are shared in whole images only)
    const bool share = inverse && blocks == cu_count() && blocks % 2 == 0 && nimg >= 2 * blocks && even_share_parts() != kEvenShareDen / 2;
    static std::atomic<unsigned long long> served[3];
    const void* fn = !inverse ? reinterpret_cast<const void*>(fft2d_trunc_kernel<LOGX, LOGY, LOGR>)
                     : share ? reinterpret_cast<const void*>(ifft2d_pad_kernel<LOGX, LOGY, true, LOGR>)
                             : reinterpret_cast<const void*>(ifft2d_pad_kernel<LOGX, LOGY, false, LOGR>);
    if (hipError_t e = allow_dynamic_lds(fn, lds_bytes, served[inverse ? (share ? 2 : 1) : 0]); e != hipSuccess) return e;
    if (share)
        hipLaunchKernelGGL((ifft2d_pad_kernel<LOGX, LOGY, true, LOGR>), dim3((unsigned)blocks), dim3(1024), lds_bytes, stream, in,
                           out, nimg, even_share_parts(), nfull);
    else if (inverse)
        hipLaunchKernelGGL((ifft2d_pad_kernel<LOGX, LOGY, false, LOGR>), dim3((unsigned)blocks), dim3(1024), lds_bytes, stream, in,
                           out, nimg, kEvenShareDen / 2, nfull);
    else
        hipLaunchKernelGGL((fft2d_trunc_kernel<LOGX, LOGY, LOGR>), dim3((unsigned)blocks), dim3(1024), lds_bytes, stream, in,
                           out, nimg, nfull);
    return hipGetLastError();
}

static hipError_t dispatch_image_kernel(bool inverse, int logDX, int logDY, const float2* in, float2* out, int nimg,
                                        hipStream_t stream)
{
    // columns: 128 or 256 rows per block, 512 / 1024 as 2 / 4 parts of 256; rows: any built length
    auto with_rows = [&](auto logy) -> hipError_t {
        constexpr int LOGY = decltype(logy)::value;
        switch (logDX) {
        case 7: return launch_image_kernel<7, LOGY, 0>(inverse, in, out, nimg, stream);
        case 8: return launch_image_kernel<8, LOGY, 0>(inverse, in, out, nimg, stream);
        case 9: return launch_image_kernel<8, LOGY, 1>(inverse, in, out, nimg, stream);
        case 10: return launch_image_kernel<8, LOGY, 2>(inverse, in, out, nimg, stream);
        default: return hipErrorInvalidValue;
        }
    };
    switch (logDY) {
    case 7: return with_rows(std::integral_constant<int, 7>{});
    case 8: return with_rows(std::integral_constant<int, 8>{});
    case 9: return with_rows(std::integral_constant<int, 9>{});
    case 10: return with_rows(std::integral_constant<int, 10>{});
    default: break;
    }
    return hipErrorInvalidValue;
}

hipError_t launch_fft2d_trunc(int logDX, int logDY, const float2* x, float2* spec, int nimg, hipStream_t stream)
{
    return dispatch_image_kernel(false, logDX, logDY, x, spec, nimg, stream);
}

hipError_t launch_ifft2d_pad(int logDX, int logDY, const float2* spec, float2* y, int nimg, hipStream_t stream)
{
    return dispatch_image_kernel(true, logDX, logDY, spec, y, nimg, stream);
}

hipError_t launch_cgemm_modes(const float2* A, const float2* W, float2* C, long Mtot, int N, int K, float2 alpha,
                              float2 beta, hipStream_t stream, int w_period)
{
    if (Mtot % 16 != 0 || Mtot <= 0 || Mtot >= (1L << 27) || N % 64 != 0 || K % 8 != 0) return hipErrorInvalidValue;
    const int Kw = w_period > 0 ? w_period : K;
    if (K % Kw != 0) return hipErrorInvalidValue;
    dim3 grid((unsigned)((Mtot + GEMM_MBLOCK - 1) / GEMM_MBLOCK), (unsigned)(N / 64), 1);
    constexpr size_t lds_bytes = sizeof(float) * 3 * kW3Plane;      // 61,632 B: above the static limit
    auto launch = [&](auto ng_const, auto multi_const) -> hipError_t {
        constexpr int NG = decltype(ng_const)::value;
        constexpr bool MULTI = decltype(multi_const)::value;
        static std::atomic<unsigned long long> served;
        if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(cgemm_modes3m_kernel<NG, MULTI>), lds_bytes, served);
            e != hipSuccess)
            return e;
        hipLaunchKernelGGL((cgemm_modes3m_kernel<NG, MULTI>), grid, dim3(GEMM_THREADS), lds_bytes, stream, A, W, C, Mtot, N, K,
                           alpha, beta, Kw);
        return hipGetLastError();
    };
    // several column blocks per CU, one chunk: persistent blocks, one per CU (and n tile)
    auto launch_persistent = [&](auto ng_const) -> hipError_t {
        constexpr int NG = decltype(ng_const)::value;
        static std::atomic<unsigned long long> served;
        if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(cgemm_modes3m_persistent_kernel<NG>), lds_bytes, served);
            e != hipSuccess)
            return e;
        const long nblocks = grid.x;
        // one block per CU and n tile; with several n tiles, 48 channels or more and up to two column blocks per CU the
        // matrix pipes are the bound and one block per CU in all is faster (N = 128, K = 64: M = 65,536 41 -> 35 us,
        // 131,072 71 -> 62; with fewer channels or more columns the kernel is bound by the loads in flight and loses 5-25 %)
        long g = cu_count();
        if (grid.y > 1 && K >= 48 && nblocks <= 2L * cu_count()) g /= (long)grid.y;
        if (g >= 8) g -= g % 8;                                  // whole groups of eight: every XCD the same share
        if (g < 1) g = 1;
        hipLaunchKernelGGL((cgemm_modes3m_persistent_kernel<NG>), dim3((unsigned)g, grid.y, 1), dim3(GEMM_THREADS), lds_bytes,
                           stream, A, W, C, Mtot, N, K, alpha, nblocks, Kw);
        return hipGetLastError();
    };
    // from two column blocks per CU (K = N = 64: M = 131,072 40 -> 37 us, 262,144 75 -> 64, 524,288 164 -> 133; below that
    // the two kernels are level)
    // Not with beta: reading C back inside the walk waits for the strip requested just before it (K = 32, M = 262,144:
    // 79 against 74 us).
    if (K <= GEMM_KC && beta.x == 0.f && beta.y == 0.f &&
        ((long)grid.x >= 2L * cu_count() || (K >= 48 && (long)grid.x * (long)grid.y >= 2L * cu_count()))) {
        if (K <= 16) return launch_persistent(std::integral_constant<int, 4>{});
        if (K <= 32) return launch_persistent(std::integral_constant<int, 8>{});
        if (K <= 48) return launch_persistent(std::integral_constant<int, 12>{});
        return launch_persistent(std::integral_constant<int, 16>{});
    }
    // from eight column blocks per CU (all n tiles together): 3-9 % ahead of the chunked kernel below (K = N = 128,
    // M = 262,144: 274 -> 255 us); level at four, and up to 8 % behind on small problems (the larger tile to build)
    if (K > GEMM_KC && K <= GEMM_KMAX && beta.x == 0.f && beta.y == 0.f && (long)grid.x * (long)grid.y >= 8L * cu_count()) {
        constexpr size_t wide_lds = sizeof(float) * 3 * kW3WidePlane;            // 123,264 B: one block per CU
        static std::atomic<unsigned long long> served;
        if (hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(cgemm_modes3m_persistent_wide_kernel), wide_lds, served);
            e != hipSuccess)
            return e;
        long g = cu_count() / (long)grid.y;
        if (g >= 8) g -= g % 8;
        if (g < 1) g = 1;
        if (g > (long)grid.x) g = grid.x;
        hipLaunchKernelGGL(cgemm_modes3m_persistent_wide_kernel, dim3((unsigned)g, grid.y, 1), dim3(GEMM_THREADS), wide_lds, stream, A,
                           W, C, Mtot, N, K, alpha, (long)grid.x, Kw);
        return hipGetLastError();
    }
    if (K <= 16) return launch(std::integral_constant<int, 4>{}, std::false_type{});
    if (K <= 32) return launch(std::integral_constant<int, 8>{}, std::false_type{});
    if (K <= 48) return launch(std::integral_constant<int, 12>{}, std::false_type{});
    if (K <= GEMM_KC) return launch(std::integral_constant<int, 16>{}, std::false_type{});
    return launch(std::integral_constant<int, 8>{}, std::true_type{});
}

}  // namespace tfno
