// Fused 1D spectral layer for SMALL grids with many channels (DY = 256): a CLUSTER of P workgroups shares one signal
// set and splits its K input channels, so that no forward transform is computed twice.
//
// Same operands and result as fused_fft_cgemm_ifft_8 of the reference
// (fusion_variants/1D_D_exp_fused_fft_cgemm_ifft/fused_fft_cgemm_ifft_7.cuh:9-222), whose (S, N/64) grid gives every
// block of a signal set ALL K forward transforms. With few signal sets (S * N/64 well below the number of CUs) that
// repetition is the critical path. Here member q of a cluster
//   1. transforms channels [q K/P, (q+1) K/P) of the signal set (32 at a time, one per 16-lane group),
//   2. multiplies them with the matching rows of W for ALL N output channels on v_mfma_f32_16x16x4_f32
//      (spectra and the real-expanded W' tile staged through LDS as in fused_fft_mfma_ifft_kernel),
//   3. publishes the partial products of the output channels it does not own to the other members through device
//      memory, keeps its own N/P channels in LDS,
//   4. waits (bounded) until all P members have published, adds the P-1 foreign partials to its own, runs the
//      zero-padded backward transforms of its N/P channels and stores y.
// Members of a cluster get block ids eight apart (same XCD, dispatched together). A waiting member only ever waits for
// blocks with ids less than 8 P away, all of which the in-order dispatcher has started or will start without this
// block's resources, whatever the grid size.
//
// Publication protocol: every partial product is one 64-bit word that says by itself whether it has been written in
// THIS launch. At the start of the kernel, long before anything is published, each consumer lane overwrites the words it
// will read at the end with a sentinel (all bits set: a NaN pattern that arithmetic on finite data never produces);
// producers later overwrite them with their partial products; the consumer reads each word until it no longer holds the
// sentinel. All of these are relaxed device-scope atomic accesses to one location each, and the argument needs nothing
// more than the coherence of a single location: the consumer's read comes after its own sentinel store in program order,
// so it returns that sentinel or a value stored later in the word's modification order - which can only be this
// launch's product (launches on a stream are ordered, a word has one producer per launch); whatever an earlier launch,
// of whatever shape, left in the buffer is wiped before it can be read. If a product lands BEFORE the sentinel (a
// consumer that started seconds after its producers), the consumer never sees it and falls back as described below:
// slow, never wrong. No ordering between different locations is needed, hence no release / acquire fences (at device
// scope those write back and invalidate the whole L2 of the XCD: +2.6 us on a 16 us kernel, measured), no counter that
// correctness depends on, and the kernel is replayable from a captured graph.
// Two counters per cluster are timing hints and nothing else. The ANNOUNCE counter guards the one weak spot of the
// scheme, a consumer that starts after its producers have published (a grid that is not resident all at once): each
// member adds to it just before it publishes its first word, and a consumer wavefront that finds it off a multiple of 8
// at its start knows that a member of this launch is already publishing; it then neither wipes nor reads but leaves its
// channels to the fallback at once instead of waiting out the bound for words it may have wiped. The ARRIVAL counter
// tells the members WHEN to read: words requested while their
// producer's stores are still on their way miss the L2 and take 3 us instead of 0.6 to come back, so each member adds
// to the counter when its own stores have completed and reads once all have done so (or 20 us have passed). The counter
// is never reset: every launch adds exactly 8 to each counter (8 / P per member), launches are ordered by their stream,
// so a member that reads the old value v knows all have arrived at (v / 8 + 1) 8. All counter accesses are relaxed; a
// counter that is early, late or out of step only costs time.
//
// Every wait is bounded. A wavefront that does not get all its words in time leaves them; when the block has stored
// what it could, it transforms the channels of the other members itself and adds their products to its own output
// channels (a plain loop, slower, same result up to summation order) and stores y again, so the output of a launch is
// valid whether or not its members ever ran side by side. Each such member counts itself in the exchange buffer, where
// turbofno_exchange_status finds the number.
//
// The exchange memory belongs to the CALLER (turbofno_exchange_attach): nothing in this file allocates, frees or
// synchronises, except that reading the status waits for the stream.
#include "group_fft.h"
#include "kernels.h"

#include <functional>
#include <map>
#include <mutex>
#include <thread>
#include <tuple>

namespace tfno {

typedef float floatx4_cl __attribute__((ext_vector_type(4)));

// NT = output channels of the layer, KC_ = channels per chunk (8, 16 or 32: lane groups that transform at a time)
template <int NT, int KC_> struct GeoCluster {
    static constexpr int KC = KC_;
    static constexpr int PA = 80, PC = 72;                      // pitches (complex) of the spectra tile and of the own product
    static constexpr int EXCH = 16 * 17;
    static constexpr int REGION0 = 32 * EXCH;                   // exchange regions (32 for the backward pass) | spectra tile sA[KC][PA]
    // W'' tile: three planes (c, d - c, c + d; alpha W = c + i d) of floats at (k / 4) * WGROUP + (k % 4) * WROW + n.
    // An operand fetch (4 k x 16 n) reads 16 consecutive floats of four rows that are 16 banks apart; the group stride
    // of 1 (mod 64 banks) spreads the tile build, whose lanes run along k, over the banks as well.
    static constexpr int WROW = NT + 16, WGROUP = 4 * WROW + 1, WPLANE = (KC / 4) * WGROUP;
    static constexpr int REGION1 = (3 * WPLANE + 1) / 2;        // complex units
    static constexpr int REGION2 = 32 * PC;                     // own product sC[<= 32][PC]
    static constexpr int TPW = NT / 32;                         // 16 n x 16 m tiles per wave (one m tile, TPW n tiles)
    static constexpr size_t LDS_BYTES = sizeof(float2) * (size_t)(REGION0 + REGION1 + REGION2);
    static_assert(KC * PA <= REGION0, "spectra tile must fit the exchange regions");
    static_assert(WROW % 64 == 16, "rows of an operand fetch must be 16 banks apart");
};

namespace {

constexpr int kArriveStride = 32;                               // counters 128 bytes apart: one line per cluster
constexpr unsigned long long kHintTicks = 2000;                 // 20 us of the 100 MHz clock: longest wait for the arrival hint
constexpr unsigned long long kUnwritten = ~0ull;               // the sentinel: both halves a NaN with all payload bits set

__device__ __forceinline__ unsigned long long load_published(const cpx* p)
{
    return __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_published(cpx* p, unsigned long long v)
{
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace

// The 4 (P - 1) words a lane reads from the other members (its channel's modes t + 16 a in each member's part).
// wipe_inbox: the sentinel over them, at the start of the kernel.
template <int P_> __device__ __forceinline__ void wipe_inbox(float2* base, long member_stride, int q)
{
#pragma unroll
    for (int qq = 1; qq < P_; ++qq) {
        float2* p = base + (long)((q + qq) & (P_ - 1)) * member_stride;
#pragma unroll
        for (int a = 0; a < 4; ++a) store_published(p + 16 * a, kUnwritten);
    }
}
// take_partials: all of them requested at once; words that still hold the sentinel are requested again until `wait_ticks`
// of the 100 MHz clock have passed. On success they are added to c. The decision is per wavefront.
template <int P_>
__device__ __forceinline__ bool take_partials(float2* base, long member_stride, int q, cpx (&c)[4], unsigned long long wait_ticks)
{
    unsigned long long f[P_ - 1][4];
#pragma unroll
    for (int qq = 1; qq < P_; ++qq) {
        float2* p = base + (long)((q + qq) & (P_ - 1)) * member_stride;
#pragma unroll
        for (int a = 0; a < 4; ++a) f[qq - 1][a] = load_published(p + 16 * a);
    }
    auto missing = [&]() {
        bool m = false;
#pragma unroll
        for (int qq = 0; qq < P_ - 1; ++qq)
#pragma unroll
            for (int a = 0; a < 4; ++a) m |= f[qq][a] == kUnwritten;
        return m;
    };
    if (__any(missing())) {
        const unsigned long long t0 = wall_clock64();
        do {
            if (wall_clock64() - t0 > wait_ticks) return false;
            __builtin_amdgcn_s_sleep(1);
#pragma unroll
            for (int qq = 1; qq < P_; ++qq) {
                float2* p = base + (long)((q + qq) & (P_ - 1)) * member_stride;
#pragma unroll
                for (int a = 0; a < 4; ++a)
                    if (f[qq - 1][a] == kUnwritten) f[qq - 1][a] = load_published(p + 16 * a);
            }
        } while (__any(missing()));
    }
#pragma unroll
    for (int qq = 0; qq < P_ - 1; ++qq)
#pragma unroll
        for (int a = 0; a < 4; ++a) c[a] = cadd(c[a], __builtin_bit_cast(cpx, f[qq][a]));
    return true;
}

// part[S][P][N][64]: partial products by (signal set, producing member), 64-bit words; arrive[S * kArriveStride]: arrival
// counters (a timing hint); *gave_up counts the members that computed the other members' share themselves.
template <int NT, int KC_>
__global__ __launch_bounds__(512) void fused_fft_mfma_ifft_cluster_kernel(int S, int K, int P, const float2* __restrict__ x,
                                                                          const float2* __restrict__ W, float2* __restrict__ y,
                                                                          float2 alpha, float2* part, unsigned* arrive,
                                                                          unsigned* gave_up, unsigned long long wait_ticks)
{
    using G = GeoCluster<NT, KC_>;
    constexpr int DY = 256, N = NT, KC = G::KC, PA = G::PA, PC = G::PC, TPW = G::TPW;
    extern __shared__ float2 lds[];
    float2* sA = lds;
    float* sW = reinterpret_cast<float*>(lds + G::REGION0);
    float2* sC = lds + G::REGION0 + G::REGION1;
    __shared__ unsigned s_late;                                 // a wavefront of this block did not get its words in time

    const int tid = threadIdx.x;
    const int g = tid >> 4, t = tid & 15;                       // transform role: lane group g, lane t
    const int wave = tid >> 6, lane = tid & 63, col = lane & 15, kq = lane >> 4;   // matrix role
    const int mt = wave & 3, tile0 = (wave >> 2) * TPW;         // m tile, first of the wave's TPW n tiles
    // block id -> (signal set, member): ids of one cluster are eight apart
    const unsigned id = blockIdx.x, j = id >> 3;
    const int q = (int)(j % (unsigned)P);
    const long s = (long)(j / (unsigned)P) * 8 + (id & 7);
    if (s >= S) return;                                         // padding of the last group of eight clusters
    const int KB = K / P, NB = N / P, kbase = q * KB;
    float2* exch = lds + g * G::EXCH;
    // The wave walks its n tiles in a rotated order that ends with the tiles this member owns: the partials of the
    // other members' channels are then on their way while the matrix cores still work on the rest.
    const int own_last = (q * NB + NB - 1) / 16;                // last tile with channels of this member
    const int rot = (own_last >= tile0 && own_last < tile0 + TPW) ? ((own_last - tile0 + 1) & (TPW - 1)) : 0;

    cpx tw[16];
    load_lane_twiddles<8>(t, tw);
    floatx4_cl p1[TPW], p2[TPW], p3[TPW];
#pragma unroll
    for (int i = 0; i < TPW; ++i) p1[i] = p2[i] = p3[i] = floatx4_cl{ 0.f, 0.f, 0.f, 0.f };

    const float2* src = x + ((long)(kbase + g) * S + s) * DY + t;
    auto issue = [&](cpx (&dst)[16], int kc) {
        const float2* p = src + (long)kc * S * DY;
#pragma unroll
        for (int i = 0; i < 16; ++i) dst[i] = p[16 * i];
    };
    cpx v[16];
    if (g < KC) issue(v, 0);
    float2* mine = part + ((long)(s * P + q) * N) * 64 + mt * 16 + col;
    // consumer role: lane group g < NB finishes output channel n; its words in the other members' parts
    const int n = NB * q + (g < NB ? g : 0);
    float2* inbox = part + ((long)s * P * N + n) * 64 + t;
    const long member_stride = (long)N * 64;
    if (tid == 0) s_late = 0;
    // W chunk: lanes run along k, the contiguous direction of W[k + n*K]; the two halves of a wavefront take channels
    // eight apart (eight banks apart in the tile)
    constexpr int WPT = KC * NT / 512;                          // KB is a multiple of KC: every chunk is full
    float2 wv[WPT];
    auto load_w = [&](int kc) {
#pragma unroll
        for (int u = 0; u < WPT; ++u) {
            const int idx = tid + u * 512;
            const int k = idx % KC, r = idx / KC, nn = (r & ~9) | ((r & 1) << 3) | ((r >> 3) & 1);
            wv[u] = W[(kbase + kc + k) + (long)nn * K];
        }
    };
    load_w(0);
    // The sentinel over the words this lane group will read at the end: behind the first loads of x and W (memory
    // results come back in the order of the requests, so no load queues up behind these stores), microseconds before
    // any member publishes - unless this block has started that late: then a member has announced itself already (the
    // counter is off a multiple of 8), and the wavefront leaves its words alone and its channels to the fallback.
    // The stores cost the kernel 0.9 us wherever they are placed (12 - 28 written-through stores per lane in the same
    // queue as the partial products); this is the place with the widest margin.
    unsigned* announce = arrive + s * kArriveStride + 1;
    bool on_time = true;                                        // uniform over the wavefront
    if (g < NB) {
        const unsigned seen = __hip_atomic_load(announce, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        on_time = (__builtin_amdgcn_readfirstlane(seen) & 7u) == 0u;
        if (on_time) {
            if (P == 2) wipe_inbox<2>(inbox, member_stride, q);
            else if (P == 4) wipe_inbox<4>(inbox, member_stride, q);
            else wipe_inbox<8>(inbox, member_stride, q);
        }
    }

    for (int kc = 0; kc < KB; kc += KC) {
        const bool last = kc + KC >= KB;
        cpx out[4];
        if (g < KC) {
            cpx gg[16];
            fwd_pass1(v, tw, gg);
            if (kc + KC < KB) issue(v, kc + KC);
            group_forward_finish<8>(gg, exch, t, out);
        }
        // W'' tile (its region is not shared with the transforms): built by whichever waves are done transforming
#pragma unroll
        for (int u = 0; u < WPT; ++u) {
            const int idx = tid + u * 512;
            const int k = idx % KC, r = idx / KC, nn = (r & ~9) | ((r & 1) << 3) | ((r >> 3) & 1);
            const float c = wv[u].x * alpha.x - wv[u].y * alpha.y, d = wv[u].x * alpha.y + wv[u].y * alpha.x;
            float* dstw = &sW[(k >> 2) * G::WGROUP + (k & 3) * G::WROW + nn];
            dstw[0] = c;
            dstw[G::WPLANE] = d - c;
            dstw[2 * G::WPLANE] = c + d;
        }
        if (!last) load_w(kc + KC);
        __syncthreads();                                        // all exchanges done: sA may overwrite them
        if (g < KC) {
#pragma unroll
            for (int a = 0; a < 4; ++a) sA[g * PA + t + 16 * a] = out[a];
        }
        __syncthreads();
        if (last && tid == 0) __hip_atomic_fetch_add(announce, 8u / (unsigned)P, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const float2* arow = sA + kq * PA + mt * 16 + col;
#pragma unroll
        for (int i = 0; i < TPW; ++i) {
            const int tile = tile0 + ((i + rot) & (TPW - 1));
            const float* wrow = sW + kq * G::WROW + tile * 16 + col;
#pragma unroll
            for (int kg = 0; kg < KC / 4; ++kg) {
                const float2 b = arow[kg * 4 * PA];
                const float* w = wrow + kg * G::WGROUP;
                p1[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[0], b.x + b.y, p1[i], 0, 0, 0);
                p2[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[G::WPLANE], b.x, p2[i], 0, 0, 0);
                p3[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[2 * G::WPLANE], b.y, p3[i], 0, 0, 0);
            }
            if (last) {
                // D[row = 4 kq + v][col]: output channel 16 tile + 4 kq + v, mode 16 mt + col. NB is a multiple of 8, so
                // the four channels of a lane have one owner.
                const int nd = 16 * tile + 4 * kq;
                const bool own = nd / NB == q;
#pragma unroll
                for (int vv = 0; vv < 4; ++vv) {
                    const float2 c = make_float2(p1[i][vv] - p3[i][vv], p1[i][vv] + p2[i][vv]);
                    if (own) sC[(nd + vv - NB * q) * PC + mt * 16 + col] = c;
                    else store_published(mine + (long)(nd + vv) * 64, __builtin_bit_cast(unsigned long long, c));
                }
            }
        }
        if (!last) __syncthreads();                             // sA / sW are free again for the next chunk
    }
    __syncthreads();                                            // the own product is complete in sC; own stores have completed
    // Arrival hint (see the head of this file): every member adds 8 / P, every launch 8 whatever its cluster size, so
    // launches with different P may follow each other on a stream; 8 divides 2^32: consistent under wrap-around.
    // A wait bound of zero means "never wait": every member then works alone, whatever the timing (the tests of that
    // path rely on it).
    if (tid == 0) {
        unsigned* ctr = arrive + s * kArriveStride;
        const unsigned add = 8u / (unsigned)P;
        const unsigned old = __hip_atomic_fetch_add(ctr, add, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned target = (old / 8u + 1u) * 8u;
        if (old + add != target && wait_ticks != 0) {
            const unsigned long long t0 = wall_clock64();
            const unsigned long long bound = wait_ticks < kHintTicks ? wait_ticks : kHintTicks;
            while ((int)(__hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - target) < 0 && wall_clock64() - t0 <= bound)
                __builtin_amdgcn_s_sleep(2);
        }
    }
    __syncthreads();

    cpx c[4];
    auto own_product = [&]() {
#pragma unroll
        for (int a = 0; a < 4; ++a) c[a] = sC[g * PC + t + 16 * a];
    };
    auto finish_channel = [&]() {                               // backward transform of channel n from c, y stored
        cpx yv[16];
        group_backward<8>(c, tw, exch, t, yv);
        float2* dst = y + ((long)n * S + s) * DY + t;
#pragma unroll
        for (int i = 0; i < 16; ++i) store_streaming(dst + 16 * i, yv[i]);
    };
    if (g < NB) {                                               // whole wavefronts: NB is a multiple of 8 lane groups
        bool ok = false;
        if (wait_ticks != 0 && on_time) {
            own_product();
            if (P == 2) ok = take_partials<2>(inbox, member_stride, q, c, wait_ticks);
            else if (P == 4) ok = take_partials<4>(inbox, member_stride, q, c, wait_ticks);
            else ok = take_partials<8>(inbox, member_stride, q, c, wait_ticks);
        }
        if (ok) finish_channel();
        else s_late = 1;
    }
    // Only when a wavefront was left without its words: the whole block computes the other members' share of the
    // contraction, for this member's output channels, from x and W. Chunks of KC channels as above (forward transforms
    // -> sA), then lane group g adds alpha W[k][n] A[k][m] over the chunk for its channel n, in the register layout the
    // backward pass takes. Every channel of the member is stored again (those that were complete get the same values up
    // to summation order).
    __syncthreads();
    if (s_late != 0) {                                          // uniform over the block
        if (tid == 0) __hip_atomic_fetch_add(gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (g < NB) own_product();
        for (int qq = 1; qq < P; ++qq) {
            const int from = (q + qq) & (P - 1);
            for (int kc = 0; kc < KB; kc += KC) {
                const int k0 = from * KB + kc;
                cpx out[4];
                if (g < KC) {
                    const float2* p = x + ((long)(k0 + g) * S + s) * DY + t;
                    cpx vv[16], gg[16];
#pragma unroll
                    for (int i = 0; i < 16; ++i) vv[i] = p[16 * i];
                    fwd_pass1(vv, tw, gg);
                    group_forward_finish<8>(gg, exch, t, out);
                }
                __syncthreads();                                // all exchanges done: sA may overwrite them
                if (g < KC) {
#pragma unroll
                    for (int a = 0; a < 4; ++a) sA[g * PA + t + 16 * a] = out[a];
                }
                __syncthreads();
                if (g < NB) {
                    for (int k = 0; k < KC; ++k) {
                        const float2 w = cmul(W[(k0 + k) + (long)n * K], alpha);
#pragma unroll
                        for (int a = 0; a < 4; ++a) c[a] = cadd(c[a], cmul(sA[k * PA + t + 16 * a], w));
                    }
                }
                __syncthreads();                                // sA is free again
            }
        }
        if (g < NB) finish_channel();
    }
}

// ------------------------------------------------------------------------------------------------------------------
// Exchange memory: caller-owned, one buffer per (device, stream), registered with exchange_attach and forgotten with a
// null attach. Layout of a buffer for a device of `cus` compute units (a clustered grid is at most one block per CU and
// N at most 128, so part[S][P][N][64] never exceeds 64 KiB per CU):
//   [0, 64 KiB * cus)                 partial products (no initial state needed: every launch wipes what it will read)
//   [.., + 128 B * cus)               arrival counters, one 128-byte line per cluster
//   [.., + 256 B)                     word 0: members that computed the others' share themselves since the last report
// Calls on one stream are ordered and share the stream's buffer; calls on different streams use different buffers.
namespace {

struct Exchange {
    float2* part = nullptr;
    unsigned* arrive = nullptr;
    unsigned* gave_up = nullptr;
    long clusters = 0;              // compute units the buffer was sized for
};

std::mutex g_exchange_mutex;
// key: device, stream handle, and - for hipStreamPerThread, one handle that names a different stream in every host
// thread - a hash of the calling thread
typedef std::tuple<int, hipStream_t, size_t> ExchangeKey;
std::map<ExchangeKey, Exchange> g_exchange;
// Default bound of a wait: 100 us of the 100 MHz wall clock, about twice what the fallback costs - waiting longer for
// members that are not running is slower than doing their work
std::atomic<unsigned long long> g_wait_ticks{ 10000ull };

constexpr size_t kPartBytesPerCu = sizeof(float2) * 64 * 128;
constexpr size_t kArriveBytesPerCu = sizeof(unsigned) * kArriveStride;
constexpr size_t kStatusBytes = 256;

bool key_of(hipStream_t stream, ExchangeKey& key)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return false; }
    const size_t thread_key = stream == hipStreamPerThread ? std::hash<std::thread::id>()(std::this_thread::get_id()) : 0;
    key = std::make_tuple(dev, stream, thread_key);
    return true;
}

bool stream_is_capturing(hipStream_t stream)
{
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &st) != hipSuccess) { (void)hipGetLastError(); return false; }
    return st != hipStreamCaptureStatusNone;
}

// stream-ordered clear (a kernel, not a memset node)
__global__ void zero_words_kernel(unsigned* p, long n)
{
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// the buffer of (current device, stream), by value; false when none is attached or it is too small for `clusters`
bool exchange_for(hipStream_t stream, long clusters, size_t bytes_per_cluster, Exchange& out)
{
    ExchangeKey key;
    if (!key_of(stream, key)) return false;
    std::lock_guard<std::mutex> lock(g_exchange_mutex);
    const auto it = g_exchange.find(key);
    if (it == g_exchange.end()) return false;
    const Exchange& e = it->second;
    if (clusters > e.clusters || (size_t)clusters * bytes_per_cluster > kPartBytesPerCu * (size_t)e.clusters) return false;
    out = e;
    return true;
}

template <int NT, int KC>
hipError_t launch_cluster_t(long S, int K, int P, const float2* x, const float2* W, float2* y, float2 alpha, const Exchange& e,
                            hipStream_t stream)
{
    using G = GeoCluster<NT, KC>;
    static std::atomic<unsigned long long> served;
    if (hipError_t err = allow_dynamic_lds(reinterpret_cast<const void*>(fused_fft_mfma_ifft_cluster_kernel<NT, KC>), G::LDS_BYTES, served);
        err != hipSuccess)
        return err;
    const long blocks = ((S + 7) / 8) * 8 * P;
    hipLaunchKernelGGL((fused_fft_mfma_ifft_cluster_kernel<NT, KC>), dim3((unsigned)blocks), dim3(512), G::LDS_BYTES, stream, (int)S, K, P,
                       x, W, y, alpha, e.part, e.arrive, e.gave_up, g_wait_ticks.load(std::memory_order_relaxed));
    return hipGetLastError();
}

}  // namespace

size_t exchange_bytes(long cus)
{
    if (cus <= 0) cus = cu_count();
    return (kPartBytesPerCu + kArriveBytesPerCu) * (size_t)cus + kStatusBytes;
}

// Registers `buffer` (exchange_bytes() bytes, 256-byte aligned, device memory of the current device) for clustered
// launches on `stream` and clears its counters with a kernel on that stream; a null buffer forgets the stream's buffer.
// hipErrorInvalidValue: misaligned or too small; hipErrorStreamCaptureUnsupported: the stream is being captured.
hipError_t exchange_attach(hipStream_t stream, void* buffer, size_t bytes)
{
    ExchangeKey key;
    if (!key_of(stream, key)) return hipErrorInvalidDevice;
    if (!buffer) {
        std::lock_guard<std::mutex> lock(g_exchange_mutex);
        g_exchange.erase(key);
        return hipSuccess;
    }
    const long cus = cu_count();
    if (((size_t)buffer & 255) || bytes < exchange_bytes(cus)) return hipErrorInvalidValue;
    if (stream_is_capturing(stream)) return hipErrorStreamCaptureUnsupported;
    Exchange e;
    e.part = static_cast<float2*>(buffer);
    e.arrive = reinterpret_cast<unsigned*>(static_cast<char*>(buffer) + kPartBytesPerCu * (size_t)cus);
    e.gave_up = reinterpret_cast<unsigned*>(static_cast<char*>(buffer) + (kPartBytesPerCu + kArriveBytesPerCu) * (size_t)cus);
    e.clusters = cus;
    const long words = (long)((kArriveBytesPerCu * (size_t)cus + kStatusBytes) / sizeof(unsigned));
    hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream, e.arrive, words);
    if (hipError_t err = hipGetLastError(); err != hipSuccess) return err;
    std::lock_guard<std::mutex> lock(g_exchange_mutex);
    g_exchange[key] = e;
    return hipSuccess;
}

bool exchange_attached(hipStream_t stream)
{
    ExchangeKey key;
    if (!key_of(stream, key)) return false;
    std::lock_guard<std::mutex> lock(g_exchange_mutex);
    return g_exchange.find(key) != g_exchange.end();
}

// Waits for the stream, then returns (and clears) the number of cluster members that have computed the other members'
// share themselves since the last call. hipErrorNotReady: no buffer attached to the stream.
hipError_t exchange_gave_up(hipStream_t stream, unsigned* count)
{
    Exchange e;
    if (!exchange_for(stream, 0, 0, e)) return hipErrorNotReady;
    unsigned host = 0;
    if (hipError_t err = hipMemcpyAsync(&host, e.gave_up, sizeof(unsigned), hipMemcpyDeviceToHost, stream); err != hipSuccess) return err;
    if (hipError_t err = hipStreamSynchronize(stream); err != hipSuccess) return err;
    if (host) {
        hipLaunchKernelGGL(zero_words_kernel, dim3(1), dim3(64), 0, stream, e.gave_up, 1L);
        if (hipError_t err = hipGetLastError(); err != hipSuccess) return err;
    }
    *count = host;
    return hipSuccess;
}

// Cluster size for (S, N, K) on `cus` compute units, or 0 when this kernel does not apply: N in {64, 128}, every member
// gets a multiple of eight input channels and 8 ... 32 output channels, and the whole grid is resident at once (one
// block per CU).
int cluster_size_1d(int logDY, long S, int N, int K, long cus)
{
    if (logDY != 8 || (N != 64 && N != 128) || S <= 0) return 0;
    const long groups = (S + 7) / 8 * 8;
    int P = 0;
    for (int c = N / 32; c <= 8; c *= 2)                        // the largest cluster that still gives every block a CU
        if (groups * c <= cus && K % (8 * c) == 0 && N / c >= 8) P = c;
    return P;
}

// hipErrorNotReady: no exchange buffer is attached to this stream (the caller falls back on a kernel without one)
hipError_t launch_fused_cluster(long S, int N, int K, int P, const float2* x, const float2* W, float2* y, float2 alpha,
                                hipStream_t stream)
{
    if (P < 2 || P > 8 || (P & (P - 1)) || K % (8 * P) || N % P || N / P > 32 || N / P < 8) return hipErrorInvalidValue;
    Exchange e;
    if (!exchange_for(stream, S, sizeof(float2) * 64 * (size_t)N * P, e)) return hipErrorNotReady;
    // chunk = the largest of 32 / 16 / 8 channels that divides a member's share
    const int KB = K / P, KC = KB % 32 == 0 ? 32 : (KB % 16 == 0 ? 16 : 8);
    if (N == 128 && KC == 32) return launch_cluster_t<128, 32>(S, K, P, x, W, y, alpha, e, stream);
    if (N == 128 && KC == 16) return launch_cluster_t<128, 16>(S, K, P, x, W, y, alpha, e, stream);
    if (N == 128) return launch_cluster_t<128, 8>(S, K, P, x, W, y, alpha, e, stream);
    if (N == 64 && KC == 32) return launch_cluster_t<64, 32>(S, K, P, x, W, y, alpha, e, stream);
    if (N == 64 && KC == 16) return launch_cluster_t<64, 16>(S, K, P, x, W, y, alpha, e, stream);
    if (N == 64) return launch_cluster_t<64, 8>(S, K, P, x, W, y, alpha, e, stream);
    return hipErrorInvalidValue;
}

void set_cluster_wait_ticks(unsigned long long ticks) { g_wait_ticks.store(ticks, std::memory_order_relaxed); }

}  // namespace tfno
