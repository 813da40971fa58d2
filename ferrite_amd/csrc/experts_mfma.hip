// Expert GEMMs on the CDNA4 block-scaled MFMA (v_mfma_scale_f32_16x16x128_f8f6f4): e2m1 weights with their
// e8m0-per-32 scales go from HBM straight into the matrix core, activations are e4m3 with e8m0-per-32 scales.
//
// Orientation: weights are the A operand (16 weight rows x 128 k per instruction), tokens are the B operand
// (16 token columns), so a unit of up to 16 tokens that share an expert streams every byte of that expert's
// weights exactly once.  Operand layouts of the instruction (measured on gfx950):
//   A (e2m1, 4 VGPRs): lane l holds row l%16, k = 32*(l/16) + [0,32), low nibble = lower k
//   B (e4m3, 8 VGPRs): lane l holds column l%16; VGPR 0-3 = k 16*(l/16) + [0,16), VGPR 4-7 = k 64 + 16*(l/16) + [0,16)
//   scale operands   : lane l, byte op_sel = e8m0 of row/column l%16 for the k block 32*(l/16) + [0,32)
//   D (f32, 4 VGPRs) : lane l, VGPR v = element (row 4*(l/16) + v, column l%16)
//
// The packed weight buffer stores, per work item (32 gate rows + the same 32 up rows, or 64 down rows), the
// code tiles in exactly the order a wave consumes them: [item][k step][tile 0..3][lane][16 B], so a wave
// reads one contiguous 4 KiB per k step with 128-bit loads; scales are [item][4 k steps][lane][tile][4 B].
#include <hip/hip_ext.h>

#include "internal.hpp"
#include "device_utils.hpp"
#include "numerics.hpp"

namespace fe {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned int u4v __attribute__((ext_vector_type(4)));  // 128-bit vector usable with nontemporal loads

static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Which main loop the 128-row units run on (a test hook, ferrite_hip_set_override): 0 = the faster one for each GEMM
// (gate/up: weights streamed into registers by blocks of 8 waves; down, whose reduction is a third as long: both
// operands staged through LDS), 1 = staged for both, 2 / 3 = streamed by blocks of 8 / 4 waves for both.
static std::atomic<int> g_prefill_variant{0};
void set_prefill_variant(int v) { g_prefill_variant.store(v, std::memory_order_relaxed); }

PackedLayout packed_layout(const ferrite_moe_shape& s) {
    PackedLayout L{};
    const size_t H = s.hidden, I = s.inter, Is = s.shared_inter, E = s.n_experts;
    auto kt4 = [](size_t K) { return (K / 128 + 3) / 4; };
    L.gu_codes_per_expert = I * H;                               // (I/32 items) * (H/128) * 4096
    L.gu_scales_per_expert = (I / 32) * kt4(H) * 1024;
    L.dn_codes_per_expert = H * I / 2;                           // (H/64 items) * (I/128) * 4096
    L.dn_scales_per_expert = (H / 64) * kt4(I) * 1024;
    size_t off = 0;
    L.gu_codes = off;  off = align_up(off + E * L.gu_codes_per_expert, 256);
    L.gu_scales = off; off = align_up(off + E * L.gu_scales_per_expert, 256);
    L.dn_codes = off;  off = align_up(off + E * L.dn_codes_per_expert, 256);
    L.dn_scales = off; off = align_up(off + E * L.dn_scales_per_expert, 256);
    L.sh_gu_codes = off;  off = align_up(off + Is * H, 256);
    L.sh_gu_scales = off; off = align_up(off + (Is / 32) * kt4(H) * 1024, 256);
    L.sh_dn_codes = off;  off = align_up(off + H * Is / 2, 256);
    L.sh_dn_scales = off; off = align_up(off + (H / 64) * kt4(Is) * 1024, 256);
    L.router_t = off; off = align_up(off + H * ((E + 63) / 64 * 64) * 4, 256);
    L.total = off;
    return L;
}

// ---- packing: a pure permutation of bytes --------------------------------------------------------
// An item covers `rpi` rows of each of `nmat` source matrices (gate_up: rpi 32, nmat 2; down: rpi 64, nmat 1);
// its 4 tiles are 16-row slices: tile -> (matrix tile / (4/nmat), rows (tile % (4/nmat))*16 ..).
struct PackSrc {
    const uint8_t* codes[2];
    const uint8_t* scales[2];
    int rows, K;       // rows per matrix, columns
    int nmat, rpi;
    size_t s_pitch;    // bytes between scale rows of the source (K/32 when dense; a loader may pad rows)
};

__global__ __launch_bounds__(256) void pack_codes_kernel(PackSrc s, int n_experts, uint4* __restrict__ dst) {
    const int KT = s.K / 128;
    const size_t items = s.rows / s.rpi;
    const size_t per_expert = items * KT * 4 * 64;  // uint4 per expert
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= per_expert * n_experts) return;
    size_t e = idx / per_expert, r = idx % per_expert;
    int lane = r & 63;
    int tile = (r >> 6) & 3;
    size_t kt = (r >> 8) % KT, item = (r >> 8) / KT;
    const int tpm = 4 / s.nmat;
    int mat = tile / tpm;
    size_t row = item * s.rpi + (size_t)(tile % tpm) * 16 + (lane & 15);
    const uint8_t* src = s.codes[mat] + (e * s.rows + row) * (s.K / 2) + kt * 64 + (lane >> 4) * 16;
    dst[idx] = *reinterpret_cast<const uint4*>(src);
}

__global__ __launch_bounds__(256) void pack_scales_kernel(PackSrc s, int n_experts, uint32_t* __restrict__ dst) {
    const int KT = s.K / 128, KT4 = (KT + 3) / 4;
    const size_t items = s.rows / s.rpi;
    const size_t per_expert = items * KT4 * 64 * 4;  // dwords per expert
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= per_expert * n_experts) return;
    size_t e = idx / per_expert, r = idx % per_expert;
    int tile = r & 3;
    int lane = (r >> 2) & 63;
    size_t k4 = (r >> 8) % KT4, item = (r >> 8) / KT4;
    const int tpm = 4 / s.nmat;
    int mat = tile / tpm;
    size_t row = item * s.rpi + (size_t)(tile % tpm) * 16 + (lane & 15);
    const uint8_t* src = s.scales[mat] + (e * s.rows + row) * s.s_pitch;
    uint32_t v = 0;
    for (int q = 0; q < 4; ++q) {
        size_t kt = k4 * 4 + q;
        uint32_t b = kt < (size_t)KT ? src[kt * 4 + (lane >> 4)] : 127u;
        v |= b << (8 * q);
    }
    dst[idx] = v;
}

// ---- the streaming core ---------------------------------------------------------------------------
// One wave, one item: for every k step, 4 A tiles from global memory (16 B per lane each), B from LDS, 4 MFMAs
// (8 with two-term activations: the same weight registers against each term's plane).
// The B operand in LDS covers one window of k steps: bq [window k steps][2][64] uint4 (the unit's activations in
// operand order), bsc [window groups of 4 k steps][64] u32 (their scales); bq2 / bsc2 the second term's plane.
struct BWindow {
    const u4v* bq;
    const u4v* bq2;
    const uint32_t* bsc;
    const uint32_t* bsc2;
};

template <int Q, bool kX2>
__device__ __forceinline__ void mfma_step(const u4v (&a)[4], const u4v& sc, const BWindow& b, uint32_t bs, uint32_t bs2,
                                          int ktw, int lane, v4f (&acc)[4]) {
    const uint32_t scs[4] = {sc[0], sc[1], sc[2], sc[3]};
    {
        const u4v b0 = b.bq[(ktw * 2 + 0) * 64 + lane];
        const u4v b1 = b.bq[(ktw * 2 + 1) * 64 + lane];
        const v8i bv = {(int)b0[0], (int)b0[1], (int)b0[2], (int)b0[3], (int)b1[0], (int)b1[1], (int)b1[2], (int)b1[3]};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const v8i av = {(int)a[t][0], (int)a[t][1], (int)a[t][2], (int)a[t][3], 0, 0, 0, 0};
            acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, acc[t], 4 /*A e2m1*/, 0 /*B e4m3*/, Q,
                                                                      (int)scs[t], Q, (int)bs);
        }
    }
    if constexpr (kX2) {
        const u4v b0 = b.bq2[(ktw * 2 + 0) * 64 + lane];
        const u4v b1 = b.bq2[(ktw * 2 + 1) * 64 + lane];
        const v8i bv = {(int)b0[0], (int)b0[1], (int)b0[2], (int)b0[3], (int)b1[0], (int)b1[1], (int)b1[2], (int)b1[3]};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const v8i av = {(int)a[t][0], (int)a[t][1], (int)a[t][2], (int)a[t][3], 0, 0, 0, 0};
            acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, acc[t], 4, 0, Q, (int)scs[t], Q, (int)bs2);
        }
    }
}

// Registers of the weight stream: two buffers of one group (4 k steps x 4 tiles) each.
struct StreamRegs {
    u4v a[2][4][4];   // [buffer][k step in group][tile]
    u4v sc[2];
};

// kKeep: plain loads, whose lines stay in the XCD's L2 for the other units of the same expert that follow this
// block; otherwise non-temporal loads, which stream about 10 % faster but are not retained.
template <bool kKeep>
__device__ __forceinline__ u4v stream_ld(const u4v* p) {
    if constexpr (kKeep) return *p;
    else return __builtin_nontemporal_load(p);
}

template <bool kKeep>
__device__ __forceinline__ void stream_load_group(StreamRegs& r, const u4v* __restrict__ wp,
                                                  const u4v* __restrict__ sp, int KT, int lane, int g4, int buf) {
    r.sc[buf] = stream_ld<kKeep>(&sp[(size_t)g4 * 64 + lane]);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int kt = g4 * 4 + q;
        if (kt < KT) {
#pragma unroll
            for (int t = 0; t < 4; ++t)
                r.a[buf][q][t] = stream_ld<kKeep>(&wp[((size_t)kt * 4 + t) * 64 + lane]);
        }
    }
}

template <bool kX2, int BUF>
__device__ __forceinline__ void stream_group(const StreamRegs& r, const BWindow& b, int KT, int g4, int g4w, int lane,
                                             v4f (&acc)[4]) {
    const uint32_t bs = b.bsc[g4w * 64 + lane];
    uint32_t bs2 = 0;
    if constexpr (kX2) bs2 = b.bsc2[g4w * 64 + lane];
    const int kt = g4 * 4, ktw = g4w * 4;
    mfma_step<0, kX2>(r.a[BUF][0], r.sc[BUF], b, bs, bs2, ktw, lane, acc);
    if (kt + 1 < KT) mfma_step<1, kX2>(r.a[BUF][1], r.sc[BUF], b, bs, bs2, ktw + 1, lane, acc);
    if (kt + 2 < KT) mfma_step<2, kX2>(r.a[BUF][2], r.sc[BUF], b, bs, bs2, ktw + 2, lane, acc);
    if (kt + 3 < KT) mfma_step<3, kX2>(r.a[BUF][3], r.sc[BUF], b, bs, bs2, ktw + 3, lane, acc);
}

// Groups [g_lo, g_hi) of the item against the window in LDS (whose first group is g_lo).  Group g_lo must already
// be in flight in buffer 0: callers issue group 0 before they fill LDS, so the first weights travel while the
// activations are staged, and every window but the last holds an even number of groups, so a window ends with the
// next one's first group in flight in buffer 0 again.  Loads run ahead to the item's last group (KT4) whatever the
// window.
template <bool kKeep, bool kX2>
__device__ __forceinline__ void stream_item(StreamRegs& r, const u4v* __restrict__ wp, const u4v* __restrict__ sp,
                                            int KT, int g_lo, int g_hi, const BWindow& b, int lane, v4f (&acc)[4]) {
    const int KT4 = (KT + 3) >> 2;
    for (int g4 = g_lo; g4 < g_hi; g4 += 2) {
        if (g4 + 1 < KT4) stream_load_group<kKeep>(r, wp, sp, KT, lane, g4 + 1, 1);
        stream_group<kX2, 0>(r, b, KT, g4, g4 - g_lo, lane, acc);
        if (g4 + 1 < g_hi) {
            if (g4 + 2 < KT4) stream_load_group<kKeep>(r, wp, sp, KT, lane, g4 + 2, 0);
            stream_group<kX2, 1>(r, b, KT, g4 + 1, g4 + 1 - g_lo, lane, acc);
        }
    }
}

// Where a unit's activations live in LDS while its weights stream past: the whole reduction length (K x 16 bytes
// per term), or windows of kWindowKt k steps.  Two-term activations of a long reduction need 2 x 16 x K bytes
// (K 4096: 128 KiB), which leaves no room for a second block on the CU; staged in windows of 2048 k they take
// 64 KiB + scales per block whatever K is.  Between two windows the block's waves meet at a barrier, refill LDS
// and meet again.  A window is a multiple of two groups (see stream_item).
constexpr int kWindowKt = 16;

// WIN: k steps per window, 0 = the whole reduction resident.
template <int WIN>
__host__ __device__ __forceinline__ int window_kt(int KT) { return WIN > 0 && KT > WIN ? WIN : KT; }
template <bool kX2, int WIN>
static inline size_t b_lds_bytes(int KT) {
    const int w = window_kt<WIN>(KT);
    return (size_t)(kX2 ? 2 : 1) * ((size_t)w * 2048 + (size_t)((w + 3) / 4) * 256);
}

// The planes of a window of w k steps at `lds`.
template <bool kX2>
struct BPlanes {
    u4v *bq, *bq2;
    uint32_t *bsc, *bsc2;
    __device__ __forceinline__ BPlanes(unsigned char* lds, int w) {
        const size_t codes = (size_t)w * 2048, scales = (size_t)((w + 3) / 4) * 256;
        bq = reinterpret_cast<u4v*>(lds);
        bq2 = kX2 ? reinterpret_cast<u4v*>(lds + codes) : nullptr;
        bsc = reinterpret_cast<uint32_t*>(lds + (kX2 ? 2 : 1) * codes);
        bsc2 = kX2 ? reinterpret_cast<uint32_t*>(lds + 2 * codes + scales) : nullptr;
    }
    __device__ __forceinline__ BWindow window() const { return BWindow{bq, bq2, bsc, bsc2}; }
};

// One 16-byte chunk / one scale word of a window: where it comes from and which slot of the B operand it fills.
// row_src(r) gives the source row of unit row r (or -1).  Source rows are `pitch` bytes apart; scale rows are in
// operand order (scale_pos), `spitch` bytes apart.
template <bool kX2>
struct BSource {
    ActPlanes src;
    size_t pitch;
    int spitch, nrows;
};

template <bool kX2, typename RowFn>
__device__ __forceinline__ int b_chunk(const BSource<kX2>& s, RowFn row_src, int kt0, int wkt, int idx, u4v& v) {
    const int chunks = wkt * 8;   // 16-byte chunks per row and plane in the window
    const int p = idx / (s.nrows * chunks), rem = idx - p * (s.nrows * chunks);
    const int c = rem / chunks, j = rem % chunks;
    const int r = row_src(c);
    const uint8_t* plane = p ? s.src.q2 : s.src.q;
    v = (u4v){0u, 0u, 0u, 0u};
    if (r >= 0) v = *reinterpret_cast<const u4v*>(plane + (size_t)r * s.pitch + (size_t)kt0 * 128 + (size_t)j * 16);
    const int ktw = j >> 3, within = (j & 7) * 16;
    const int half = within >> 6, g = (within & 63) >> 4;
    return (p << 30) | ((ktw * 2 + half) * 64 + g * 16 + c);
}

template <bool kX2, typename RowFn>
__device__ __forceinline__ int b_scale_word(const BSource<kX2>& s, RowFn row_src, int kt0, int wkt, int idx, uint32_t& v) {
    const int wg = (wkt + 3) / 4;
    const int p = idx / (wg * 64), rem = idx - p * (wg * 64);
    const int k4 = rem >> 6, l = rem & 63, c = l & 15, g = l >> 4;
    v = 0x7f7f7f7fu;
    if (c < s.nrows) {
        const int r = row_src(c);
        const uint8_t* plane = p ? s.src.s2 : s.src.s;
        if (r >= 0) v = *reinterpret_cast<const uint32_t*>(plane + (size_t)r * s.spitch + (kt0 / 4 + k4) * 16 + g * 4);
    }
    return (p << 30) | rem;
}

// Copies k steps [kt0, kt0 + wkt) of the unit's rows into LDS in B-operand order and builds the packed scale words
// (any window length; loads and stores alternate).
template <bool kX2, typename RowFn>
__device__ __forceinline__ void fill_b_window(const BSource<kX2>& s, RowFn row_src, int kt0, int wkt,
                                              const BPlanes<kX2>& d) {
    constexpr int NP = kX2 ? 2 : 1;
    const int total = NP * s.nrows * wkt * 8;
    for (int idx = threadIdx.x; idx < total; idx += blockDim.x) {
        u4v v;
        const int slot = b_chunk<kX2>(s, row_src, kt0, wkt, idx, v);
        ((slot >> 30) ? d.bq2 : d.bq)[slot & 0x3fffffff] = v;
    }
    const int wg = (wkt + 3) / 4;
    for (int idx = threadIdx.x; idx < NP * wg * 64; idx += blockDim.x) {
        uint32_t v;
        const int slot = b_scale_word<kX2>(s, row_src, kt0, wkt, idx, v);
        ((slot >> 30) ? d.bsc2 : d.bsc)[slot & 0x3fffffff] = v;
    }
}

// The reduction of `rounds` items per wave against one unit's activation rows.  item(round, wp, sp) gives the
// round's weight stream of this wave (false: no item, the wave only keeps the barriers company); the first round's
// group 0 must already be in flight in buffer 0.  done(round, acc) receives the finished accumulators.  Every wave of the block makes the same calls: the barriers inside are block-wide.
template <bool kKeep, bool kX2, int WIN, typename RowFn, typename ItemFn, typename DoneFn>
__device__ __forceinline__ void run_unit(const BSource<kX2>& s, RowFn row_src, int KT, int rounds, ItemFn item, DoneFn done,
                                         StreamRegs& regs, unsigned char* lds, int lane) {
    const int WKT = window_kt<WIN>(KT), nw = (KT + WKT - 1) / WKT;
    const BPlanes<kX2> d(lds, WKT);
    const BWindow win = d.window();
    bool filled = false;
#pragma unroll 1
    for (int r = 0; r < rounds; ++r) {
        const u4v *wp, *sp;
        const bool live = item(r, wp, sp);
        if (r > 0 && live) stream_load_group<kKeep>(regs, wp, sp, KT, lane, 0, 0);
        v4f acc[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[t] = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
        for (int w = 0; w < nw; ++w) {
            const int kt0 = w * WKT, wkt = min(WKT, KT - kt0);
            if (nw > 1 || !filled) {
                if (filled) __syncthreads();   // every wave is done with the window that is in LDS
                fill_b_window<kX2>(s, row_src, kt0, wkt, d);
                __syncthreads();
                filled = true;
            }
            if (live) stream_item<kKeep, kX2>(regs, wp, sp, KT, kt0 / 4, (kt0 + wkt + 3) / 4, win, lane, acc);
        }
        if (live) done(r, acc);
    }
}

struct MfmaArgs {
    const uint8_t* codes;         // routed experts
    const uint8_t* scales;
    const uint8_t* sh_codes;      // shared expert
    const uint8_t* sh_scales;
    size_t codes_per_expert, scales_per_expert;
    const int32_t *unit_expert, *unit_row0, *unit_rows, *unit_first, *unit_count, *n_units;
    int n, topk, n_experts, hidden, inter, shared_inter, act_ld, unit_cap, max_units;
    float limit;
};

// A unit read from device tables is used only if it is well formed.
__device__ __forceinline__ bool unit_ok(const MfmaArgs& a, int e, int row0, int nrows) {
    const int nk = a.n * a.topk;
    if (nrows < 1 || nrows > a.unit_cap || row0 < 0) return false;
    if (e == a.n_experts) return a.shared_inter > 0 && row0 >= nk && row0 + nrows <= nk + a.n;
    return e >= 0 && e < a.n_experts && row0 + nrows <= nk;
}

// Block -> (unit, item group).  Hardware deals consecutive blocks round-robin over the 8 XCDs; the live work
// (n_units * groups) is cut into 8 contiguous ranges, one per XCD, so that the blocks of one expert share an L2.
// Within a range the order is (expert, item group, unit of the expert): the units of an expert that need the
// same weight tiles are dispatched back to back, run in lockstep and fetch those tiles from HBM once (with the
// units of an expert a whole item-group sweep apart, or on different XCDs, each of them fetched them again).
// Used by the 128-row kernels (2-3 units per expert) and by the 16-row kernels (the shared expert's n/16 units, an
// expert with more than 16 rows).  Returns false for blocks without work or with inconsistent tables.
__device__ __forceinline__ bool unit_block_work(const MfmaArgs& a, int groups, int& u, int& ig, int& ne) {
    const int n_units = min(*a.n_units, a.max_units);
    const int total = n_units * groups, per_xcd = (total + 7) >> 3;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int v = xcd * per_xcd + slot;
    if (slot >= per_xcd || v >= total) return false;
    const int up = v / groups;                       // some unit of the expert whose segment holds v
    const int first = a.unit_first[up];
    ne = a.unit_count[up];
    if (first < 0 || ne < 1 || up < first || up >= first + ne || first + ne > n_units) return false;
    const int vl = v - first * groups;               // 0 .. ne * groups - 1
    ig = vl / ne;
    u = first + (vl - ig * ne);
    return true;
}

// gate/up GEMM + clamped SwiGLU + e4m3-per-32 quantisation of the result (one or two terms).
// grid: unit_block_work over groups = ceil(items / WAVES) item groups; wave w of item group ig owns item
// ig*WAVES + w of the unit's expert.
// The unit (expert e, activation rows row0 .. row0 + nrows - 1, whose tokens row_src(c) names) against item group ig.
template <int WAVES, bool kKeep, bool kX2, int WIN, typename RowFn>
__device__ __forceinline__ void gate_up_rows(const MfmaArgs& a, int e, int row0, int nrows, int ig, RowFn row_src,
                                             const ActPlanes& xin, const ActPlanes& act, unsigned char* lds_raw) {
    const bool shared = e == a.n_experts;
    const int inter = shared ? a.shared_inter : a.inter;
    const int items = inter / 32;
    if (ig * WAVES >= items) return;
    const int H = a.hidden, KT = H / 128, KT4 = (KT + 3) / 4;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int item = ig * WAVES + wave;
    const bool live = item < items;
    const uint8_t* cbase = shared ? a.sh_codes : a.codes + (size_t)e * a.codes_per_expert;
    const uint8_t* sbase = shared ? a.sh_scales : a.scales + (size_t)e * a.scales_per_expert;
    const u4v* wp0 = reinterpret_cast<const u4v*>(cbase) + (size_t)item * KT * 256;
    const u4v* sp0 = reinterpret_cast<const u4v*>(sbase) + (size_t)item * KT4 * 64;
    StreamRegs regs;
    if (live) {   // weights fly while the activations are staged
        stream_load_group<kKeep>(regs, wp0, sp0, KT, lane, 0, 0);
    }
    const BSource<kX2> bsrc{xin, (size_t)H, scale_pitch(H), nrows};
    run_unit<kKeep, kX2, WIN>(
        bsrc, row_src, KT, 1,
        [&](int, const u4v*& wp, const u4v*& sp) { wp = wp0; sp = sp0; return live; },
        [&](int, v4f (&acc)[4]) {
            // tiles 0,1 = gate rows [0,16),[16,32) of the item; tiles 2,3 = the same up rows
            float r0[4], r1[4];
            float amax = 0.0f;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                r0[v] = swiglu_fast(acc[0][v], acc[2][v], a.limit);
                r1[v] = swiglu_fast(acc[1][v], acc[3][v], a.limit);
                amax = fmaxf(amax, fmaxf(fabsf(r0[v]), fabsf(r1[v])));
            }
            amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
            amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
            const int c = lane & 15, g = lane >> 4;
            const uint32_t sb = block_scale_e8m0(amax);
            const float inv = u2f((254u - sb) << 23);
            const uint32_t p0 = e4m3_encode4_hw(r0[0] * inv, r0[1] * inv, r0[2] * inv, r0[3] * inv);
            const uint32_t p1 = e4m3_encode4_hw(r1[0] * inv, r1[1] * inv, r1[2] * inv, r1[3] * inv);
            const size_t qoff = (size_t)(row0 + c) * a.act_ld + (size_t)item * 32 + g * 4;
            const size_t soff = (size_t)(row0 + c) * scale_pitch(a.act_ld) + scale_pos(item);
            if (c < nrows) {
                *reinterpret_cast<uint32_t*>(act.q + qoff) = p0;
                *reinterpret_cast<uint32_t*>(act.q + qoff + 16) = p1;
                if (g == 0) act.s[soff] = (uint8_t)sb;
            }
            if constexpr (kX2) {
                // second term: the same quantiser on what the first leaves over
                const float sc = u2f(sb << 23);
                float amax2 = 0.0f;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    r0[v] = fadd(r0[v], -fmul(e4m3_decode((p0 >> (8 * v)) & 0xffu), sc));
                    r1[v] = fadd(r1[v], -fmul(e4m3_decode((p1 >> (8 * v)) & 0xffu), sc));
                    amax2 = fmaxf(amax2, fmaxf(fabsf(r0[v]), fabsf(r1[v])));
                }
                amax2 = fmaxf(amax2, __shfl_xor(amax2, 16, 64));
                amax2 = fmaxf(amax2, __shfl_xor(amax2, 32, 64));
                const uint32_t sb2 = block_scale_e8m0(amax2);
                const float inv2 = u2f((254u - sb2) << 23);
                const uint32_t t0 = e4m3_encode4_hw(r0[0] * inv2, r0[1] * inv2, r0[2] * inv2, r0[3] * inv2);
                const uint32_t t1 = e4m3_encode4_hw(r1[0] * inv2, r1[1] * inv2, r1[2] * inv2, r1[3] * inv2);
                if (c < nrows) {
                    *reinterpret_cast<uint32_t*>(act.q2 + qoff) = t0;
                    *reinterpret_cast<uint32_t*>(act.q2 + qoff + 16) = t1;
                    if (g == 0) act.s2[soff] = (uint8_t)sb2;
                }
            }
        },
        regs, lds_raw, lane);
}

template <int WAVES, bool kKeep, bool kX2, int WIN>
__device__ __forceinline__ void gate_up_unit(const MfmaArgs& a, int u, int ig, const ActPlanes& xin,
                                             const int32_t* __restrict__ gather_src, const ActPlanes& act,
                                             unsigned char* lds_raw) {
    const int e = a.unit_expert[u], row0 = a.unit_row0[u], nrows = a.unit_rows[u];
    if (!unit_ok(a, e, row0, nrows)) return;   // tables from an uninitialised workspace must not cause a fault
    const bool shared = e == a.n_experts;
    const int nk = a.n * a.topk, topk = a.topk;
    gate_up_rows<WAVES, kKeep, kX2, WIN>(
        a, e, row0, nrows, ig,
        [&](int c) -> int {
            int g = row0 + c;
            if (shared) return g - nk;
            int i = gather_src[g];
            return (i < 0 || i >= nk) ? -1 : i / topk;
        },
        xin, act, lds_raw);
}

// WIN: window of the activation staging in k steps, 0 = resident (see window_kt).  One-term activations are always
// resident; two-term ones are windowed at 2048 k with two 4-wave blocks per CU, or resident with one 8-wave block
// per CU (the launcher chooses).
template <int WAVES, bool kX2, int WIN>
__global__ __launch_bounds__(WAVES * 64, WAVES == 4 ? 2 : 1) void gate_up_mfma_kernel(MfmaArgs a, int groups, ActPlanes xin,
                                                                                      const int32_t* __restrict__ gather_src,
                                                                                      ActPlanes act) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    int u, ig, ne;
    if (!unit_block_work(a, groups, u, ig, ne)) return;
    // an expert with several units: its weights are wanted again by the blocks that follow on this XCD
    if (ne > 1) gate_up_unit<WAVES, true, kX2, WIN>(a, u, ig, xin, gather_src, act, lds_raw);
    else gate_up_unit<WAVES, false, kX2, WIN>(a, u, ig, xin, gather_src, act, lds_raw);
}

// down GEMM: y[row][h] for the unit's rows.  grid: unit_block_work over groups = ceil(items / (WAVES*IPW)); item =
// 64 rows of H.
template <int WAVES, int IPW, bool kKeep, bool kX2>
__device__ __forceinline__ void down_unit(const MfmaArgs& a, int u, int ig, const ActPlanes& act, float* __restrict__ y,
                                          unsigned char* lds_raw) {
    const int e = a.unit_expert[u], row0 = a.unit_row0[u], nrows = a.unit_rows[u];
    if (!unit_ok(a, e, row0, nrows)) return;
    const bool shared = e == a.n_experts;
    const int inter = shared ? a.shared_inter : a.inter;
    const int H = a.hidden, items = H / 64;
    const int KT = inter / 128, KT4 = (KT + 3) / 4;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int item0 = (ig * WAVES + wave) * IPW;
    const uint8_t* cbase = shared ? a.sh_codes : a.codes + (size_t)e * a.codes_per_expert;
    const uint8_t* sbase = shared ? a.sh_scales : a.scales + (size_t)e * a.scales_per_expert;
    StreamRegs regs;
    if (item0 < items) {   // the first item's weights fly while the activations are staged
        const u4v* wp0 = reinterpret_cast<const u4v*>(cbase) + (size_t)item0 * KT * 256;
        const u4v* sp0 = reinterpret_cast<const u4v*>(sbase) + (size_t)item0 * KT4 * 64;
        stream_load_group<kKeep>(regs, wp0, sp0, KT, lane, 0, 0);
    }
    // activation rows have pitch act_ld; only the first `inter` columns are meaningful for this expert
    const BSource<kX2> bsrc{act, (size_t)a.act_ld, scale_pitch(a.act_ld), nrows};
    const int c = lane & 15, g = lane >> 4;
    run_unit<kKeep, kX2, kX2 ? kWindowKt : 0>(
        bsrc, [&](int col) { return row0 + col; }, KT, IPW,
        [&](int r, const u4v*& wp, const u4v*& sp) {
            const int item = item0 + r;
            wp = reinterpret_cast<const u4v*>(cbase) + (size_t)item * KT * 256;
            sp = reinterpret_cast<const u4v*>(sbase) + (size_t)item * KT4 * 64;
            return item < items;
        },
        [&](int r, v4f (&acc)[4]) {
            if (c < nrows) {
                float* dst = y + (size_t)(row0 + c) * H + (size_t)(item0 + r) * 64 + g * 4;
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    *reinterpret_cast<float4*>(dst + t * 16) = make_float4(acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
            }
        },
        regs, lds_raw, lane);
}

template <int WAVES, int IPW, bool kX2>
__global__ __launch_bounds__(WAVES * 64, 2) void down_mfma_kernel(MfmaArgs a, int groups, ActPlanes act,
                                                               float* __restrict__ y) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    int u, ig, ne;
    if (!unit_block_work(a, groups, u, ig, ne)) return;
    if (ne > 1) down_unit<WAVES, IPW, true, kX2>(a, u, ig, act, y, lds_raw);
    else down_unit<WAVES, IPW, false, kX2>(a, u, ig, act, y, lds_raw);
}


// ---- prefill kernels: units of up to 128 rows ------------------------------------------------------------
// One block (4 waves) computes 4 items (128 gate + 128 up rows, or 256 down rows) x 128 grouped rows of one unit.
// Both operands go through LDS, one k step (128 k) per stage, two stages, filled by direct global->LDS loads
// (global_load_lds_dwordx4: lane l of the issuing wave lands at base + 16*l, so the lane -> source address map
// alone produces the operand order; no staging registers, no LDS write instructions).  Wave w fills item w and
// row tiles 2w, 2w+1 of the next stage while the MFMAs of the current one run; it computes items 2*(w&1),
// 2*(w&1)+1 x rows 64*(w>>1) .. +63: 8 weight tiles x 4 row tiles = 32 MFMAs per k step.  128 accumulator
// registers + <= 128 others let two blocks share a CU, so one block's stage hand-over (wait for the loads,
// barrier, operand reads) hides behind the other's MFMAs.
// Accumulation order over k is the same as in the 16-row kernels, so both give the same bits.
constexpr int PF_ROWS = 128;
constexpr int PF_ROWS_X2 = 64;                         // two-term activations: half the rows, both planes of each
constexpr int PF_ITEMS = 4;                            // 8 (one block of 8 waves per CU) is correct too and measured slower
constexpr int PF_WAVES = PF_ITEMS;                     // one wave per item for the fills; 2 items x 64 rows each for the MFMAs
constexpr int PF_A_SLOTS = PF_ITEMS * 256;             // u4v of weights per stage
constexpr int PF_LDS_STAGE = PF_A_SLOTS + 1024;        // + 1024 activation slots
constexpr size_t PF_LDS_BYTES = 2 * PF_LDS_STAGE * 16;  // 64 KiB (4 items) / 96 KiB (8 items)

typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void glb_void;

// 16 bytes per lane from global memory straight into LDS at lds_base + 16 * lane (lds_base wave-uniform).
__device__ __forceinline__ void dma16(const void* g, void* lds_base) {
    __builtin_amdgcn_global_load_lds((glb_void*)g, (lds_void*)lds_base, 16, 0, 0);
}

struct PfCtx {
    const u4v* a_src;         // codes of the item this wave stages, k step 0, + lane
    const uint8_t* b_src[2];  // e4m3 rows (2*wave+i)*16 + lane/4 of the unit, + the lane's 16-byte chunk
    const u4v* asp[2];        // weight scale words of the wave's two items
    const uint8_t* bsp[4];    // activation scale rows of the lane's column in the wave's 4 row tiles
    int KT, wave, wi, wt, lane, bslot;
    int ntile;                // row tiles of this wave that hold rows of the unit (0..4): the others get no MFMAs
};

// Starts the loads of k step kt into `stage`.
__device__ __forceinline__ void pf_fill(const PfCtx& c, u4v* stage, int kt) {
    const u4v* a = c.a_src + (size_t)kt * 256;
#pragma unroll
    for (int t = 0; t < 4; ++t) dma16(a + t * 64, stage + (c.wave * 4 + t) * 64);
    constexpr int NB = 16 / PF_WAVES;   // half tiles of activations per wave
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int i = j >> 1, h = j & 1;   // NB 4: tiles 2w, 2w+1 x halves; NB 2: tile w x halves
        dma16(c.b_src[i] + (size_t)kt * 128 + h * 64, stage + PF_A_SLOTS + (c.wave * NB + j) * 64);
    }
}

// All loads into LDS issued by this wave have landed (vmcnt 0; expcnt and lgkmcnt left alone).
__device__ __forceinline__ void pf_wait_fill() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// One k step: operands of the current stage into registers, then the next stage's loads are started (after the
// operand reads in program order: the compiler cannot tell the two stages apart and would otherwise wait for the
// loads before it reads), then the MFMAs; the step ends when the next stage is complete for every wave.
template <int Q>
__device__ __forceinline__ void pf_step(const PfCtx& c, u4v* lds, int kt, const u4v (&asc)[2],
                                        const uint32_t (&bsc)[4], v4f (&acc)[2][4][4]) {
    const u4v* cur = lds + (Q & 1) * PF_LDS_STAGE;
    v8i bv[4];
    u4v av[2][4];
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
        const u4v* bt = cur + PF_A_SLOTS + (c.wt * 4 + tt) * 128 + c.bslot;
        const u4v b0 = bt[0];
        const u4v b1 = bt[64];
        bv[tt] = (v8i){(int)b0[0], (int)b0[1], (int)b0[2], (int)b0[3], (int)b1[0], (int)b1[1], (int)b1[2], (int)b1[3]};
    }
#pragma unroll
    for (int ii = 0; ii < 2; ++ii)
#pragma unroll
        for (int t = 0; t < 4; ++t) av[ii][t] = cur[((c.wi * 2 + ii) * 4 + t) * 64 + c.lane];
    __builtin_amdgcn_sched_barrier(0);
    pf_fill(c, lds + ((Q + 1) & 1) * PF_LDS_STAGE, min(kt + 1, c.KT - 1));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
        if (tt >= c.ntile) break;   // wave-uniform: a unit's last block of rows is usually far from full
#pragma unroll
        for (int ii = 0; ii < 2; ++ii) {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const v8i a8 = {(int)av[ii][t][0], (int)av[ii][t][1], (int)av[ii][t][2], (int)av[ii][t][3], 0, 0, 0, 0};
                acc[ii][t][tt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                    a8, bv[tt], acc[ii][t][tt], 4 /*A e2m1*/, 0 /*B e4m3*/, Q, (int)asc[ii][t], Q, (int)bsc[tt]);
            }
        }
    }
    __builtin_amdgcn_sched_barrier(0);   // the MFMAs stay in front of the wait: they are what hides the loads
    pf_wait_fill();
    __syncthreads();
}

__device__ __forceinline__ void pf_load_scales(const PfCtx& c, int g4, u4v (&asc)[2], uint32_t (&bsc)[4]) {
    const int g = c.lane >> 4;
#pragma unroll
    for (int ii = 0; ii < 2; ++ii) asc[ii] = c.asp[ii][(size_t)g4 * 64 + c.lane];
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) bsc[tt] = *reinterpret_cast<const uint32_t*>(c.bsp[tt] + g4 * 16 + g * 4);
}

__device__ __forceinline__ void pf_mainloop(const PfCtx& c, u4v* lds, v4f (&acc)[2][4][4]) {
    const int KT4 = (c.KT + 3) >> 2, full = c.KT >> 2;
    pf_fill(c, lds, 0);
    u4v asc[2], asc_n[2];
    uint32_t bsc[4], bsc_n[4];
    pf_load_scales(c, 0, asc, bsc);
#pragma unroll
    for (int ii = 0; ii < 2; ++ii)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int tt = 0; tt < 4; ++tt) acc[ii][t][tt] = (v4f){0.f, 0.f, 0.f, 0.f};
    pf_wait_fill();
    __syncthreads();
#pragma unroll 1
    for (int g4 = 0; g4 < full; ++g4) {
        pf_load_scales(c, min(g4 + 1, KT4 - 1), asc_n, bsc_n);
        const int kt = g4 * 4;
        pf_step<0>(c, lds, kt, asc, bsc, acc);
        pf_step<1>(c, lds, kt + 1, asc, bsc, acc);
        pf_step<2>(c, lds, kt + 2, asc, bsc, acc);
        pf_step<3>(c, lds, kt + 3, asc, bsc, acc);
#pragma unroll
        for (int ii = 0; ii < 2; ++ii) asc[ii] = asc_n[ii];
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) bsc[tt] = bsc_n[tt];
    }
    // k steps beyond the last full group of four (block-uniform branches)
    const int kt = full * 4, rem = c.KT & 3;
    if (rem > 0) pf_step<0>(c, lds, kt, asc, bsc, acc);
    if (rem > 1) pf_step<1>(c, lds, kt + 1, asc, bsc, acc);
    if (rem > 2) pf_step<2>(c, lds, kt + 2, asc, bsc, acc);
}

// Fills the context.  row_q(c) returns the e4m3 row of unit column c, row_s(c) its scale row; columns >= nrows
// alias column 0 (their results are never stored).
template <typename RowQ, typename RowS>
__device__ __forceinline__ void pf_context(PfCtx& c, const uint8_t* cbase, const uint8_t* sbase, int item0, int items,
                                           int KT, int nrows, RowQ row_q, RowS row_s) {
    const int KT4 = (KT + 3) >> 2;
    c.KT = KT;
    c.lane = threadIdx.x & 63;
    c.wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    c.wi = c.wave % (PF_ITEMS / 2); c.wt = c.wave / (PF_ITEMS / 2);
    c.ntile = min(4, max(0, (nrows - c.wt * 64 + 15) >> 4));
    const int cc = c.lane & 15, g = c.lane >> 4;
    c.a_src = reinterpret_cast<const u4v*>(cbase) + (size_t)min(item0 + c.wave, items - 1) * KT * 256 + c.lane;
    // Activation stage layout: the four lanes of a quad fetch 64 consecutive bytes of one row (what the texture
    // addresser coalesces), so row r's 16-byte chunk q of a half k step lands at slot 4r + q; the chunk a lane
    // fetches is XORed with (r/2)%4 so that any eight consecutive lanes of the operand read (rows r..r+7 at a fixed
    // chunk) touch eight different 16-byte bank groups (counters: no LDS bank conflicts; XOR with r/4 had them).
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int col = (PF_WAVES == 4 ? c.wave * 2 + i : c.wave) * 16 + (c.lane >> 2);
        c.b_src[i] = row_q(col < nrows ? col : 0) + ((c.lane & 3) ^ ((c.lane >> 3) & 3)) * 16;
    }
    c.bslot = 4 * cc + (g ^ ((cc >> 1) & 3));
#pragma unroll
    for (int ii = 0; ii < 2; ++ii) {
        const int item = min(item0 + c.wi * 2 + ii, items - 1);
        c.asp[ii] = reinterpret_cast<const u4v*>(sbase) + (size_t)item * KT4 * 64;
    }
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
        const int col = (c.wt * 4 + tt) * 16 + cc;
        c.bsp[tt] = row_s(col < nrows ? col : 0);
    }
}

__global__ __launch_bounds__(PF_WAVES * 64, PF_WAVES == 4 ? 2 : 1) void gate_up_prefill_kernel(MfmaArgs a, int groups, const uint8_t* __restrict__ xq,
                                                              const uint8_t* __restrict__ xs,
                                                              const int32_t* __restrict__ gather_src,
                                                              uint8_t* __restrict__ act_q,
                                                              uint8_t* __restrict__ act_s) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    int u, ig, ne;
    if (!unit_block_work(a, groups, u, ig, ne)) return;
    const int e = a.unit_expert[u], row0 = a.unit_row0[u], nrows = a.unit_rows[u];
    if (!unit_ok(a, e, row0, nrows)) return;
    const bool shared = e == a.n_experts;
    const int inter = shared ? a.shared_inter : a.inter;
    const int items = inter / 32, item0 = ig * PF_ITEMS;
    if (item0 >= items) return;
    const int H = a.hidden, nk = a.n * a.topk, topk = a.topk, n = a.n;
    const int spitch = scale_pitch(H);
    auto token = [&](int col) -> int {
        const int gr = row0 + col;
        if (shared) return gr - nk;
        const int i = gather_src[gr];
        const int tk = (i < 0 || i >= nk) ? 0 : i / topk;
        return tk < n ? tk : 0;
    };
    PfCtx c;
    pf_context(c, shared ? a.sh_codes : a.codes + (size_t)e * a.codes_per_expert,
               shared ? a.sh_scales : a.scales + (size_t)e * a.scales_per_expert, item0, items, H / 128, nrows,
               [&](int col) { return xq + (size_t)token(col) * H; },
               [&](int col) { return xs + (size_t)token(col) * spitch; });
    v4f acc[2][4][4];
    pf_mainloop(c, reinterpret_cast<u4v*>(lds_raw), acc);

    const int cc = c.lane & 15, g = c.lane >> 4;
    const int apitch = scale_pitch(a.act_ld);
#pragma unroll
    for (int ii = 0; ii < 2; ++ii) {
        const int item = item0 + c.wi * 2 + ii;
        if (item >= items) break;
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            const int col = (c.wt * 4 + tt) * 16 + cc;
            float r0[4], r1[4];
            float amax = 0.0f;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                r0[v] = swiglu_fast(acc[ii][0][tt][v], acc[ii][2][tt][v], a.limit);
                r1[v] = swiglu_fast(acc[ii][1][tt][v], acc[ii][3][tt][v], a.limit);
                amax = fmaxf(amax, fmaxf(fabsf(r0[v]), fabsf(r1[v])));
            }
            amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
            amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
            if (col < nrows) {
                const uint32_t sb = block_scale_e8m0(amax);
                const float inv = u2f((254u - sb) << 23);
                const uint32_t p0 = e4m3_encode4_hw(r0[0] * inv, r0[1] * inv, r0[2] * inv, r0[3] * inv);
                const uint32_t p1 = e4m3_encode4_hw(r1[0] * inv, r1[1] * inv, r1[2] * inv, r1[3] * inv);
                uint8_t* dst = act_q + (size_t)(row0 + col) * a.act_ld + (size_t)item * 32 + g * 4;
                *reinterpret_cast<uint32_t*>(dst) = p0;
                *reinterpret_cast<uint32_t*>(dst + 16) = p1;
                if (g == 0) act_s[(size_t)(row0 + col) * apitch + scale_pos(item)] = (uint8_t)sb;
            }
        }
    }
}

// Two f32 -> two bf16 in one dword, round to nearest even (v_cvt_pk_bf16_f32; NaN stays NaN).
__device__ __forceinline__ uint32_t bf16_pk(float lo, float hi) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    const f2 v = {lo, hi};
    const bf2 h = __builtin_convertvector(v, bf2);
    return *reinterpret_cast<const uint32_t*>(&h);
}

// Writes the bf16 form of 16 rows x 64 columns of y (one item's columns for one tile of rows): r[t] holds, for the
// lane's row c = lane % 16, columns 16 t + 4 g .. + 3 with g = lane / 16, as the MFMA leaves them.  Stored from
// there, a wave's store instruction would put 8 bytes per lane, four 8-byte pieces 32 bytes apart in each of 16
// rows, and the memory pipeline takes as long per such piece as per full line: at 4096 tokens the stores of
// the 128-row down kernel cost 83 us of its 291 us.  So the pieces change lanes first: two lane-row swaps
// (v_permlane32_swap, v_permlane16_swap) per dword pair hand lane (c, g) the 16 bytes at columns 8 g and the 16
// bytes at columns 32 + 8 g of its row, then neighbouring rows trade their second halves (DPP quad_perm), and each
// of the two store instructions writes eight whole 128-byte rows: 243 us.  `y_row0` points at column 0 of the item
// in the row of c = 0; rows c >= rows_here are not written.  Every lane of the wave must call this.
__device__ __forceinline__ void store_y_tile_bf16(uint16_t* __restrict__ y_row0, size_t pitch, int rows_here, v4f r0,
                                                  v4f r1, v4f r2, v4f r3, int lane) {
    typedef unsigned u2v __attribute__((ext_vector_type(2)));
    const int c = lane & 15, g = lane >> 4;
    uint32_t lo[4] = {bf16_pk(r0[0], r0[1]), bf16_pk(r1[0], r1[1]), bf16_pk(r2[0], r2[1]), bf16_pk(r3[0], r3[1])};
    uint32_t hi[4] = {bf16_pk(r0[2], r0[3]), bf16_pk(r1[2], r1[3]), bf16_pk(r2[2], r2[3]), bf16_pk(r3[2], r3[3])};
    // lane rows g = 0..3 of registers (t, t+1): [t0 t1 t2 t3] [u0 u1 u2 u3] -> [t0 t2 u0 u2] [t1 t3 u1 u3]
#pragma unroll
    for (int p = 0; p < 4; p += 2) {
        u2v a = __builtin_amdgcn_permlane32_swap(lo[p], lo[p + 1], false, false);
        a = __builtin_amdgcn_permlane16_swap(a[0], a[1], false, false);
        u2v b = __builtin_amdgcn_permlane32_swap(hi[p], hi[p + 1], false, false);
        b = __builtin_amdgcn_permlane16_swap(b[0], b[1], false, false);
        lo[p] = a[0]; lo[p + 1] = a[1]; hi[p] = b[0]; hi[p + 1] = b[1];
    }
    // now (lo[0], hi[0], lo[1], hi[1]) = columns 8 g .. 8 g + 7 and (lo[2], hi[2], lo[3], hi[3]) = columns 32 + 8 g ..
    const uint32_t q0 = __builtin_amdgcn_update_dpp(0u, lo[2], 0xB1, 0xf, 0xf, false);   // lane ^ 1's second half
    const uint32_t q1 = __builtin_amdgcn_update_dpp(0u, hi[2], 0xB1, 0xf, 0xf, false);
    const uint32_t q2 = __builtin_amdgcn_update_dpp(0u, lo[3], 0xB1, 0xf, 0xf, false);
    const uint32_t q3 = __builtin_amdgcn_update_dpp(0u, hi[3], 0xB1, 0xf, 0xf, false);
    const bool even = (c & 1) == 0;
    // first store: the even row of each pair, its first half from the even lane, its second half from the odd lane
    const u4v sa = {even ? lo[0] : q0, even ? hi[0] : q1, even ? lo[1] : q2, even ? hi[1] : q3};
    const u4v sb = {even ? q0 : lo[0], even ? q1 : hi[0], even ? q2 : lo[1], even ? q3 : hi[1]};
    const int ra = c & ~1, rb = c | 1;
    const int first = g * 8, second = 32 + g * 8;
    if (ra < rows_here) *reinterpret_cast<u4v*>(y_row0 + (size_t)ra * pitch + (even ? first : second)) = sa;
    if (rb < rows_here) *reinterpret_cast<u4v*>(y_row0 + (size_t)rb * pitch + (even ? second : first)) = sb;
}

template <typename YT>
__global__ __launch_bounds__(PF_WAVES * 64, PF_WAVES == 4 ? 2 : 1) void down_prefill_kernel(MfmaArgs a, int groups, const uint8_t* __restrict__ act_q,
                                                           const uint8_t* __restrict__ act_s, YT* __restrict__ y) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    int u, ig, ne;
    if (!unit_block_work(a, groups, u, ig, ne)) return;
    const int e = a.unit_expert[u], row0 = a.unit_row0[u], nrows = a.unit_rows[u];
    if (!unit_ok(a, e, row0, nrows)) return;
    const bool shared = e == a.n_experts;
    const int inter = shared ? a.shared_inter : a.inter;
    const int H = a.hidden, items = H / 64, item0 = ig * PF_ITEMS;
    if (item0 >= items) return;
    const int apitch = scale_pitch(a.act_ld), act_ld = a.act_ld;
    PfCtx c;
    pf_context(c, shared ? a.sh_codes : a.codes + (size_t)e * a.codes_per_expert,
               shared ? a.sh_scales : a.scales + (size_t)e * a.scales_per_expert, item0, items, inter / 128, nrows,
               [&](int col) { return act_q + (size_t)(row0 + col) * act_ld; },
               [&](int col) { return act_s + (size_t)(row0 + col) * apitch; });
    v4f acc[2][4][4];
    pf_mainloop(c, reinterpret_cast<u4v*>(lds_raw), acc);

    const int cc = c.lane & 15, g = c.lane >> 4;
#pragma unroll
    for (int ii = 0; ii < 2; ++ii) {
        const int item = item0 + c.wi * 2 + ii;
        if (item >= items) break;
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            const int tile0 = (c.wt * 4 + tt) * 16;
            if constexpr (sizeof(YT) == 4) {
                const int col = tile0 + cc;
                if (col < nrows) {
                    YT* dst = y + (size_t)(row0 + col) * H + (size_t)item * 64 + g * 4;
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const v4f r = acc[ii][t][tt];
                        *reinterpret_cast<float4*>(dst + t * 16) = make_float4(r[0], r[1], r[2], r[3]);
                    }
                }
            } else {
                store_y_tile_bf16(y + (size_t)(row0 + tile0) * H + (size_t)item * 64, (size_t)H, nrows - tile0,
                                  acc[ii][0][tt], acc[ii][1][tt], acc[ii][2][tt], acc[ii][3][tt], c.lane);
            }
        }
    }
}

// ---- prefill kernels, weight-streaming form --------------------------------------------------------------
// One block (W waves) computes W items x NT*16 grouped rows of one unit.  Wave w owns item w for all of the rows:
// its weights go from global memory straight into registers, 16 bytes per lane and tile as in the 16-row kernels,
// through a ring of three k steps, so that a k step's tiles were asked for two to three steps before they are
// used: far enough ahead for HBM.  Only the activations are shared by the block's waves and go through LDS: a ring
// of three stages of one k step each ([tile][half][64 lanes] 16-byte slots in the operand order and slot swizzle
// of the LDS-staged kernels, then [tile][64 lanes] scale words), filled through registers (ordinary loads keep the
// compiler's wait counts exact, which loads that write LDS directly do not): the loads of step k+2 are issued at
// the top of step k, written to their stage at the top of step k+1 and read during step k+2, one barrier per step.
// Accumulation order over k is that of the other kernels: the same bits.
template <int W, int NT>
struct StCfg {
    static constexpr int STAGES = 3;
    static constexpr int CODE_SLOTS = NT * 128;            // 16-byte slots of e4m3 codes per stage
    static constexpr int STAGE_SLOTS = CODE_SLOTS + NT * 16;   // + NT * 64 scale words
    static constexpr size_t LDS_BYTES = (size_t)STAGES * STAGE_SLOTS * 16;
    static constexpr int CF = 2 * NT / W;                  // 1 KiB pieces of codes per wave and stage
    static constexpr int SF = (NT + W - 1) / W;            // 256-byte pieces of scale words per wave and stage
    static_assert((2 * NT) % W == 0, "the code pieces of a stage must divide among the waves");
};

// All four streams of a block are read through buffer resources (a wave-uniform base in scalar registers, a 32-bit
// byte offset per lane that does not change over k, and the k step as a scalar offset): no 64-bit address
// arithmetic in vector registers, of which this kernel has none to spare, and reads past a stream's end return 0.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void* base, size_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)(bytes > 0xffffffffull ? 0xffffffffull : bytes),
                                             0x00020000);
}
__device__ __forceinline__ u4v rsrc_ld16(rsrc_t r, uint32_t voff, uint32_t soff) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0);
}
__device__ __forceinline__ uint32_t rsrc_ld4(rsrc_t r, uint32_t voff, uint32_t soff) {
    return __builtin_amdgcn_raw_buffer_load_b32(r, (int)voff, (int)soff, 0);
}

template <int W, int NT>
struct StCtx {
    rsrc_t ra, ras;          // this wave's item: codes [KT][4 tiles][64 lanes][16 B], scale words [KT4][64 lanes][16 B]
    rsrc_t rb, rbs;          // activation codes and scale rows (operand order)
    uint32_t aoff;           // 16 * lane
    uint32_t coff[StCfg<W, NT>::CF];   // byte offset of the lane's chunk of piece i at k step 0
    uint32_t soff[StCfg<W, NT>::SF];   // byte offset of the lane's scale word of piece i, group 0
    int KT, lane, wave, ntile, bslot;
};

// A stage holds NT operand tiles of 16 rows each.  With one-term activations tile v is rows 16 v .. 16 v + 15 of the
// unit; with two-term activations (P = 2 planes) the unit has NT / 2 tiles of rows and tile v is plane v % 2 of row
// tile v / 2: both planes of a row tile accumulate into the same registers, and the tiles that hold rows of the unit
// are the first ones of the stage in either case.
// row_q(v, r) / row_s(v, r): byte offsets of row r of tile v's code row / scale row from bq / bs.
template <int P, int W, int NT, typename RowQ, typename RowS>
__device__ __forceinline__ void st_context(StCtx<W, NT>& c, const uint8_t* cbase, const uint8_t* sbase, int item, int KT,
                                           int nrows, const uint8_t* bq, size_t bq_bytes, const uint8_t* bs,
                                           size_t bs_bytes, RowQ row_q, RowS row_s) {
    using Cfg = StCfg<W, NT>;
    const int KT4 = (KT + 3) >> 2;
    c.KT = KT;
    c.lane = threadIdx.x & 63;
    c.wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    c.ntile = min(NT / P, (nrows + 15) >> 4);
    c.ra = make_rsrc(cbase + (size_t)item * KT * 4096, (size_t)KT * 4096);
    c.ras = make_rsrc(sbase + (size_t)item * KT4 * 1024, (size_t)KT4 * 1024);
    c.rb = make_rsrc(bq, bq_bytes);
    c.rbs = make_rsrc(bs, bs_bytes);
    c.aoff = (uint32_t)c.lane * 16;
    const int cc = c.lane & 15, g = c.lane >> 4;
    // piece j of a stage = (tile j/2, half j%2): the four lanes of a quad fetch 64 consecutive bytes of row lane/4 of
    // the tile, the chunk a lane fetches XORed with (row/2)%4 (see pf_context)
#pragma unroll
    for (int i = 0; i < Cfg::CF; ++i) {
        const int j = c.wave * Cfg::CF + i;
        c.coff[i] = row_q(j >> 1, c.lane >> 2) + (uint32_t)((j & 1) * 64 + ((c.lane & 3) ^ ((c.lane >> 3) & 3)) * 16);
    }
#pragma unroll
    for (int i = 0; i < Cfg::SF; ++i) c.soff[i] = row_s(min(c.wave * Cfg::SF + i, NT - 1), cc) + (uint32_t)(g * 4);
    c.bslot = 4 * cc + (g ^ ((cc >> 1) & 3));
}

template <int W, int NT>
struct StFill {
    u4v cr[StCfg<W, NT>::CF];
    uint32_t sr[StCfg<W, NT>::SF];
};

template <int W, int NT>
__device__ __forceinline__ void st_load(const StCtx<W, NT>& c, int kt, StFill<W, NT>& f) {
#pragma unroll
    for (int i = 0; i < StCfg<W, NT>::CF; ++i) f.cr[i] = rsrc_ld16(c.rb, c.coff[i], (uint32_t)kt * 128);
#pragma unroll
    for (int i = 0; i < StCfg<W, NT>::SF; ++i) f.sr[i] = rsrc_ld4(c.rbs, c.soff[i], (uint32_t)(kt >> 2) * 16);
}

template <int W, int NT>
__device__ __forceinline__ void st_store(const StCtx<W, NT>& c, u4v* stage, const StFill<W, NT>& f) {
    using Cfg = StCfg<W, NT>;
#pragma unroll
    for (int i = 0; i < Cfg::CF; ++i) stage[(c.wave * Cfg::CF + i) * 64 + c.lane] = f.cr[i];
    uint32_t* sw = reinterpret_cast<uint32_t*>(stage + Cfg::CODE_SLOTS);
#pragma unroll
    for (int i = 0; i < Cfg::SF; ++i)
        if (c.wave * Cfg::SF + i < NT) sw[(c.wave * Cfg::SF + i) * 64 + c.lane] = f.sr[i];
}

// The weights of k step kt (4 tiles) and the scale words of its group of four k steps.
struct StWeights {
    u4v a[4];
    u4v sc;
};

template <int W, int NT>
__device__ __forceinline__ void st_load_a(const StCtx<W, NT>& c, int kt, StWeights& w) {
#pragma unroll
    for (int t = 0; t < 4; ++t) w.a[t] = rsrc_ld16(c.ra, c.aoff + t * 1024, (uint32_t)kt * 4096);
    w.sc = rsrc_ld16(c.ras, c.aoff, (uint32_t)(kt >> 2) * 1024);
}

// k step kt against stage R = kt % 3 of the ring, with the weights in ring slot R.  The scale operands select their
// byte with op_sel 0: the words are shifted by the k step's byte (kt % 4) first, which leaves the unrolling free
// to follow the rings.  Every load is issued whatever kt is (past the end the last k step is fetched again and never
// used): a load behind a branch makes the compiler wait for all loads at the next use of any.
// kFull: all NT tiles of rows are live; otherwise tiles beyond ntile get no MFMAs (a unit's last block of rows is
// usually far from full).
template <int R, bool kFull, int P, int W, int NT>
__device__ __forceinline__ void st_step(const StCtx<W, NT>& c, u4v* lds, int kt, StWeights (&w)[3], StFill<W, NT>& f,
                                        v4f (&acc)[4][NT / P]) {
    using Cfg = StCfg<W, NT>;
    __syncthreads();   // stage R is complete; nobody reads the stage that is written next any more
    st_store(c, lds + ((R + 1) % 3) * Cfg::STAGE_SLOTS, f);
    __builtin_amdgcn_sched_barrier(0);
    st_load(c, min(kt + 2, c.KT - 1), f);
    __builtin_amdgcn_sched_barrier(0);
    const u4v* stage = lds + R * Cfg::STAGE_SLOTS;
    const uint32_t* sw = reinterpret_cast<const uint32_t*>(stage + Cfg::CODE_SLOTS);
    const int sh = (kt & 3) * 8;
#pragma unroll
    for (int t = 0; t < 4; ++t) w[R].sc[t] >>= sh;   // in place: a slot's scale words are used by this step only
    // operand registers of the row tiles: two sets used in turn (a tile is read while the MFMAs of the tile before
    // it run), or one where registers are short (the other wave of the SIMD then covers the read)
    constexpr int NB = W * NT <= 32 ? 1 : 2;
    u4v b[NB][2];
    uint32_t bs[NB];
    auto read_tile = [&](int tt) {
        const u4v* bt = stage + tt * 128 + c.bslot;
        b[tt % NB][0] = bt[0];
        b[tt % NB][1] = bt[64];
        bs[tt % NB] = sw[tt * 64 + c.lane];
    };
    read_tile(0);
#pragma unroll
    for (int tt = 0; tt < NT; ++tt) {
        const int rt = tt / P;
        if (kFull || rt < c.ntile) {   // block-uniform; the live tiles are the first ones
            if (NB == 2 && tt + 1 < NT) read_tile(tt + 1);
            const u4v b0 = b[tt % NB][0], b1 = b[tt % NB][1];
            bs[tt % NB] >>= sh;
            const v8i bv = {(int)b0[0], (int)b0[1], (int)b0[2], (int)b0[3], (int)b1[0], (int)b1[1], (int)b1[2], (int)b1[3]};
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const v8i a8 = {(int)w[R].a[t][0], (int)w[R].a[t][1], (int)w[R].a[t][2], (int)w[R].a[t][3], 0, 0, 0, 0};
                acc[t][rt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, bv, acc[t][rt], 4 /*A e2m1*/, 0 /*B e4m3*/,
                                                                              0, (int)w[R].sc[t], 0, (int)bs[tt % NB]);
            }
            if (NB == 1 && tt + 1 < NT) read_tile(tt + 1);
            // Pins the tile: its MFMAs stay in front of this point and the operand reads of the tiles after the next
            // behind it.  Without it the compiler reads all tiles of the step first (64 more registers than there are).
            asm volatile("" : "+v"(acc[0][rt]), "+v"(acc[1][rt]), "+v"(acc[2][rt]), "+v"(acc[3][rt]) : : "memory");
        }
    }
    st_load_a(c, min(kt + 3, c.KT - 1), w[R]);
    __builtin_amdgcn_sched_barrier(0);
}

template <bool kFull, int P, int W, int NT>
__device__ __forceinline__ void st_steps(const StCtx<W, NT>& c, u4v* lds, StWeights (&w)[3], StFill<W, NT>& f,
                                         v4f (&acc)[4][NT / P]) {
    const int KT = c.KT;
    int kt = 0;
#pragma unroll 1
    for (; kt + 3 <= KT; kt += 3) {
        st_step<0, kFull, P>(c, lds, kt, w, f, acc);
        st_step<1, kFull, P>(c, lds, kt + 1, w, f, acc);
        st_step<2, kFull, P>(c, lds, kt + 2, w, f, acc);
    }
    const int rem = KT - kt;   // block-uniform
    if (rem > 0) st_step<0, kFull, P>(c, lds, kt, w, f, acc);
    if (rem > 1) st_step<1, kFull, P>(c, lds, kt + 1, w, f, acc);
}

template <int P, int W, int NT>
__device__ __forceinline__ void st_mainloop(const StCtx<W, NT>& c, u4v* lds, v4f (&acc)[4][NT / P]) {
    const int KT = c.KT;
    StWeights w[3];
#pragma unroll
    for (int q = 0; q < 3; ++q) st_load_a(c, min(q, KT - 1), w[q]);
    StFill<W, NT> f;
    st_load(c, 0, f);
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int tt = 0; tt < NT / P; ++tt) acc[t][tt] = (v4f){0.f, 0.f, 0.f, 0.f};
    st_store(c, lds, f);
    st_load(c, min(1, KT - 1), f);
    st_steps<false, P>(c, lds, w, f, acc);
}

// The span of two planes that one buffer resource covers: plane p starts d[p] bytes after lo.
struct PlaneSpan {
    const uint8_t* lo;
    uint32_t d0, d1;
    size_t bytes;
    __device__ __forceinline__ uint32_t at(int plane) const { return plane ? d1 : d0; }
};
__device__ __forceinline__ PlaneSpan plane_span(const uint8_t* p0, const uint8_t* p1, size_t plane_bytes) {
    if (!p1) return PlaneSpan{p0, 0u, 0u, plane_bytes};
    const uint8_t* lo = p0 < p1 ? p0 : p1;
    const uint32_t d0 = (uint32_t)(p0 - lo), d1 = (uint32_t)(p1 - lo);
    return PlaneSpan{lo, d0, d1, (size_t)(d0 > d1 ? d0 : d1) + plane_bytes};
}

// P = 1: one-term activations, units of up to NT * 16 rows.  P = 2: two-term activations (both planes of x in, both
// planes of the SwiGLU output out), units of up to NT * 8 rows: per k step and tile of rows a second MFMA against
// the second plane with the same weight registers, so the stage, the fills and the MFMAs per block are those of
// P = 1 and a launch has twice the blocks.
template <int W, int NT, int P>
__global__ __launch_bounds__(W * 64, W * NT <= 32 ? 2 : 1) void gate_up_stream_kernel(
    MfmaArgs a, int groups, ActPlanes xin, const int32_t* __restrict__ gather_src, ActPlanes act) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    constexpr int RT = NT / P;
    int u, ig, ne;
    if (!unit_block_work(a, groups, u, ig, ne)) return;
    const int e = a.unit_expert[u], row0 = a.unit_row0[u], nrows = a.unit_rows[u];
    if (!unit_ok(a, e, row0, nrows)) return;
    const bool shared = e == a.n_experts;
    const int inter = shared ? a.shared_inter : a.inter;
    const int items = inter / 32, item0 = ig * W;
    if (item0 >= items) return;
    const int H = a.hidden, nk = a.n * a.topk, topk = a.topk, n = a.n;
    const int spitch = scale_pitch(H);
    auto token = [&](int col) -> int {
        const int gr = row0 + (col < nrows ? col : 0);
        if (shared) return gr - nk;
        const int i = gather_src[gr];
        const int tk = (i < 0 || i >= nk) ? 0 : i / topk;
        return tk < n ? tk : 0;
    };
    const PlaneSpan xq = plane_span(xin.q, P == 2 ? xin.q2 : nullptr, (size_t)n * H);
    const PlaneSpan xs = plane_span(xin.s, P == 2 ? xin.s2 : nullptr, (size_t)n * spitch);
    StCtx<W, NT> c;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int item = item0 + wave;
    st_context<P>(c, shared ? a.sh_codes : a.codes + (size_t)e * a.codes_per_expert,
                  shared ? a.sh_scales : a.scales + (size_t)e * a.scales_per_expert, min(item, items - 1), H / 128, nrows,
                  xq.lo, xq.bytes, xs.lo, xs.bytes,
                  [&](int v, int r) { return xq.at(v % P) + (uint32_t)token((v / P) * 16 + r) * (uint32_t)H; },
                  [&](int v, int r) { return xs.at(v % P) + (uint32_t)token((v / P) * 16 + r) * (uint32_t)spitch; });
    v4f acc[4][RT];
    st_mainloop<P>(c, reinterpret_cast<u4v*>(lds_raw), acc);
    if (item >= items) return;

    // tiles 0,1 = gate rows [0,16),[16,32) of the item; tiles 2,3 = the same up rows
    const int cc = c.lane & 15, g = c.lane >> 4;
    const int apitch = scale_pitch(a.act_ld);
#pragma unroll
    for (int tt = 0; tt < RT; ++tt) {
        if (tt >= c.ntile) continue;
        const int col = tt * 16 + cc;
        float r0[4], r1[4];
        float amax = 0.0f;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            r0[v] = swiglu_fast(acc[0][tt][v], acc[2][tt][v], a.limit);
            r1[v] = swiglu_fast(acc[1][tt][v], acc[3][tt][v], a.limit);
            amax = fmaxf(amax, fmaxf(fabsf(r0[v]), fabsf(r1[v])));
        }
        amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
        amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
        const uint32_t sb = block_scale_e8m0(amax);
        const float inv = u2f((254u - sb) << 23);
        const uint32_t p0 = e4m3_encode4_hw(r0[0] * inv, r0[1] * inv, r0[2] * inv, r0[3] * inv);
        const uint32_t p1 = e4m3_encode4_hw(r1[0] * inv, r1[1] * inv, r1[2] * inv, r1[3] * inv);
        const size_t qoff = (size_t)(row0 + col) * a.act_ld + (size_t)item * 32 + g * 4;
        const size_t soff = (size_t)(row0 + col) * apitch + scale_pos(item);
        if (col < nrows) {
            *reinterpret_cast<uint32_t*>(act.q + qoff) = p0;
            *reinterpret_cast<uint32_t*>(act.q + qoff + 16) = p1;
            if (g == 0) act.s[soff] = (uint8_t)sb;
        }
        if constexpr (P == 2) {
            // second term: the same quantiser on what the first leaves over (as in the 16-row kernel)
            const float sc = u2f(sb << 23);
            float amax2 = 0.0f;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                r0[v] = fadd(r0[v], -fmul(e4m3_decode((p0 >> (8 * v)) & 0xffu), sc));
                r1[v] = fadd(r1[v], -fmul(e4m3_decode((p1 >> (8 * v)) & 0xffu), sc));
                amax2 = fmaxf(amax2, fmaxf(fabsf(r0[v]), fabsf(r1[v])));
            }
            amax2 = fmaxf(amax2, __shfl_xor(amax2, 16, 64));
            amax2 = fmaxf(amax2, __shfl_xor(amax2, 32, 64));
            const uint32_t sb2 = block_scale_e8m0(amax2);
            const float inv2 = u2f((254u - sb2) << 23);
            const uint32_t t0 = e4m3_encode4_hw(r0[0] * inv2, r0[1] * inv2, r0[2] * inv2, r0[3] * inv2);
            const uint32_t t1 = e4m3_encode4_hw(r1[0] * inv2, r1[1] * inv2, r1[2] * inv2, r1[3] * inv2);
            if (col < nrows) {
                *reinterpret_cast<uint32_t*>(act.q2 + qoff) = t0;
                *reinterpret_cast<uint32_t*>(act.q2 + qoff + 16) = t1;
                if (g == 0) act.s2[soff] = (uint8_t)sb2;
            }
        }
    }
}

template <int W, int NT, int P, typename YT>
__global__ __launch_bounds__(W * 64, W * NT <= 32 ? 2 : 1) void down_stream_kernel(MfmaArgs a, int groups, ActPlanes act,
                                                                                   YT* __restrict__ y) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    constexpr int RT = NT / P;
    int u, ig, ne;
    if (!unit_block_work(a, groups, u, ig, ne)) return;
    const int e = a.unit_expert[u], row0 = a.unit_row0[u], nrows = a.unit_rows[u];
    if (!unit_ok(a, e, row0, nrows)) return;
    const bool shared = e == a.n_experts;
    const int inter = shared ? a.shared_inter : a.inter;
    const int H = a.hidden, items = H / 64, item0 = ig * W;
    if (item0 >= items) return;
    const int apitch = scale_pitch(a.act_ld), act_ld = a.act_ld;
    // both planes from the unit's first row on: the resources end with the unit's last row
    const PlaneSpan aq = plane_span(act.q + (size_t)row0 * act_ld, P == 2 ? act.q2 + (size_t)row0 * act_ld : nullptr,
                                    (size_t)nrows * act_ld);
    const PlaneSpan as = plane_span(act.s + (size_t)row0 * apitch, P == 2 ? act.s2 + (size_t)row0 * apitch : nullptr,
                                    (size_t)nrows * apitch);
    StCtx<W, NT> c;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int item = item0 + wave;
    auto rowc = [&](int v, int r) { const int col = (v / P) * 16 + r; return (uint32_t)(col < nrows ? col : 0); };
    st_context<P>(c, shared ? a.sh_codes : a.codes + (size_t)e * a.codes_per_expert,
                  shared ? a.sh_scales : a.scales + (size_t)e * a.scales_per_expert, min(item, items - 1), inter / 128, nrows,
                  aq.lo, aq.bytes, as.lo, as.bytes,
                  [&](int v, int r) { return aq.at(v % P) + rowc(v, r) * (uint32_t)act_ld; },
                  [&](int v, int r) { return as.at(v % P) + rowc(v, r) * (uint32_t)apitch; });
    v4f acc[4][RT];
    st_mainloop<P>(c, reinterpret_cast<u4v*>(lds_raw), acc);
    if (item >= items) return;

    const int cc = c.lane & 15, g = c.lane >> 4;
#pragma unroll
    for (int tt = 0; tt < RT; ++tt) {
        if (tt >= c.ntile) continue;
        if constexpr (sizeof(YT) == 4) {
            const int col = tt * 16 + cc;
            if (col < nrows) {
                YT* dst = y + (size_t)(row0 + col) * H + (size_t)item * 64 + g * 4;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const v4f r = acc[t][tt];
                    *reinterpret_cast<float4*>(dst + t * 16) = make_float4(r[0], r[1], r[2], r[3]);
                }
            }
        } else {
            store_y_tile_bf16(y + (size_t)(row0 + tt * 16) * H + (size_t)item * 64, (size_t)H, nrows - tt * 16, acc[0][tt],
                              acc[1][tt], acc[2][tt], acc[3][tt], c.lane);
        }
    }
}

// ---- launchers ----------------------------------------------------------------------------------------
// true when two planes of `bytes` each can be addressed from the lower one with 32-bit offsets
static bool planes_within_4g(const uint8_t* p0, const uint8_t* p1, size_t bytes) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(p0), b = reinterpret_cast<uintptr_t>(p1);
    return (a > b ? a - b : b - a) + bytes < 0xffffffffull;
}

constexpr int GU_WAVES = 4;
constexpr int GU_WAVES_RESIDENT_X2 = 8;
constexpr int DN_WAVES = 4;
constexpr int DN_IPW = 2;

static MfmaArgs make_args(const ferrite_moe_shape& s, const uint8_t* packed, int n, const UnitTables& units, bool down) {
    PackedLayout L = packed_layout(s);
    MfmaArgs a{};
    a.codes = packed + (down ? L.dn_codes : L.gu_codes);
    a.scales = packed + (down ? L.dn_scales : L.gu_scales);
    a.sh_codes = packed + (down ? L.sh_dn_codes : L.sh_gu_codes);
    a.sh_scales = packed + (down ? L.sh_dn_scales : L.sh_gu_scales);
    a.codes_per_expert = down ? L.dn_codes_per_expert : L.gu_codes_per_expert;
    a.scales_per_expert = down ? L.dn_scales_per_expert : L.gu_scales_per_expert;
    a.unit_expert = units.unit_expert; a.unit_row0 = units.unit_row0; a.unit_rows = units.unit_rows;
    a.unit_first = units.unit_first; a.unit_count = units.unit_count;
    a.n_units = units.n_units;
    a.n = n; a.topk = s.topk; a.n_experts = s.n_experts; a.hidden = s.hidden; a.inter = s.inter;
    a.shared_inter = s.shared_inter;
    a.act_ld = s.inter > s.shared_inter ? s.inter : s.shared_inter;
    a.limit = s.swiglu_limit;
    a.unit_cap = units.unit_rows_cap;
    a.max_units = units.max_units;
    return a;
}

// k_start / k_stop (may be null): events that bracket the kernel itself on the device, not the launch.
int launch_gate_up_mfma(const ferrite_moe_shape& s, const uint8_t* packed, const ActPlanes& xin, int n,
                        const int32_t* gather_src, const UnitTables& units, const ActPlanes& act, hipStream_t st,
                        hipEvent_t k_start, hipEvent_t k_stop) {
    MfmaArgs a = make_args(s, packed, n, units, false);
    const int imax = a.act_ld;
    const bool x2 = xin.q2 != nullptr;
    if (x2 != (act.q2 != nullptr)) return FERRITE_ERR_INVALID_ARG;
    if (units.unit_rows_cap >= PF_ROWS_X2) {
        // the tiled kernels: 128-row units of one-term activations, 64-row units of two-term activations
        if (units.unit_rows_cap != (x2 ? PF_ROWS_X2 : PF_ROWS)) return FERRITE_ERR_INVALID_ARG;
        const int variant = g_prefill_variant.load(std::memory_order_relaxed);
        auto go = [&](auto kernel, int W, size_t lds) -> int {
            const int groups = (imax / 32 + W - 1) / W;
            const unsigned blocks = (unsigned)(((size_t)units.max_units * groups + 7) / 8 * 8);
            hipExtLaunchKernelGGL(kernel, dim3(blocks), dim3(W * 64), (uint32_t)lds, st, k_start, k_stop, 0, a, groups,
                                  xin, gather_src, act);
            return check_launch("gate_up_stream");
        };
        int rc;
        if (x2) {
            // both planes through one buffer resource each: 32-bit offsets
            if (!planes_within_4g(xin.q, xin.q2, (size_t)n * s.hidden) || !planes_within_4g(xin.s, xin.s2, (size_t)n * scale_pitch(s.hidden)))
                return FERRITE_ERR_INVALID_ARG;
            if ((rc = LdsLimit<&gate_up_stream_kernel<8, 8, 2>>::ensure(StCfg<8, 8>::LDS_BYTES))) return rc;
            return go(gate_up_stream_kernel<8, 8, 2>, 8, StCfg<8, 8>::LDS_BYTES);
        }
        if (variant == 3) {
            if ((rc = LdsLimit<&gate_up_stream_kernel<4, 8, 1>>::ensure(StCfg<4, 8>::LDS_BYTES))) return rc;
            return go(gate_up_stream_kernel<4, 8, 1>, 4, StCfg<4, 8>::LDS_BYTES);
        }
        if (variant != 1) {
            if ((rc = LdsLimit<&gate_up_stream_kernel<8, 8, 1>>::ensure(StCfg<8, 8>::LDS_BYTES))) return rc;
            return go(gate_up_stream_kernel<8, 8, 1>, 8, StCfg<8, 8>::LDS_BYTES);
        }
        const int groups = (imax / 32 + PF_ITEMS - 1) / PF_ITEMS;
        const unsigned blocks = (unsigned)(((size_t)units.max_units * groups + 7) / 8 * 8);
        if ((rc = LdsLimit<&gate_up_prefill_kernel>::ensure(PF_LDS_BYTES))) return rc;
        hipExtLaunchKernelGGL(gate_up_prefill_kernel, dim3(blocks), dim3(PF_WAVES * 64), (uint32_t)PF_LDS_BYTES, st, k_start,
                              k_stop, 0, a, groups, xin.q, xin.s, gather_src, act.q, act.s);
        return check_launch("gate_up_prefill");
    }
    if (units.unit_rows_cap != 16) return FERRITE_ERR_INVALID_ARG;
    const int KT = s.hidden / 128;
    int rc;
    if (x2) {
        // Two-term activations of 16 rows take 2 x 16 x H bytes.  Where that fits LDS and an expert sees more than a
        // few rows, one 8-wave block per CU keeps them resident; otherwise 2048-k windows and two 4-wave blocks per
        // CU (the windows' barriers cost less than the lost second block when units are nearly empty, more when
        // they are full: 32 tokens 125 / 130 us, 192 tokens 178 / 168 us at H 4096).
        const size_t lds_res = b_lds_bytes<true, 0>(KT);
        const bool resident = lds_res <= kLdsCap && (long)n * s.topk > 4L * s.n_experts && KT > kWindowKt;
        if (resident) {
            constexpr int W = GU_WAVES_RESIDENT_X2;
            const int groups = (imax / 32 + W - 1) / W;
            const unsigned blocks = (unsigned)(((size_t)units.max_units * groups + 7) / 8 * 8);
            if ((rc = LdsLimit<&gate_up_mfma_kernel<W, true, 0>>::ensure(lds_res))) return rc;
            hipExtLaunchKernelGGL((gate_up_mfma_kernel<W, true, 0>), dim3(blocks), dim3(W * 64), (uint32_t)lds_res, st,
                                  k_start, k_stop, 0, a, groups, xin, gather_src, act);
        } else {
            const size_t lds = b_lds_bytes<true, kWindowKt>(KT);
            const int groups = (imax / 32 + GU_WAVES - 1) / GU_WAVES;
            const unsigned blocks = (unsigned)(((size_t)units.max_units * groups + 7) / 8 * 8);
            if ((rc = LdsLimit<&gate_up_mfma_kernel<GU_WAVES, true, kWindowKt>>::ensure(lds))) return rc;
            hipExtLaunchKernelGGL((gate_up_mfma_kernel<GU_WAVES, true, kWindowKt>), dim3(blocks), dim3(GU_WAVES * 64),
                                  (uint32_t)lds, st, k_start, k_stop, 0, a, groups, xin, gather_src, act);
        }
    } else {
        const size_t lds = b_lds_bytes<false, 0>(KT);
        const int groups = (imax / 32 + GU_WAVES - 1) / GU_WAVES;
        const unsigned blocks = (unsigned)(((size_t)units.max_units * groups + 7) / 8 * 8);
        if ((rc = LdsLimit<&gate_up_mfma_kernel<GU_WAVES, false, 0>>::ensure(lds))) return rc;
        hipExtLaunchKernelGGL((gate_up_mfma_kernel<GU_WAVES, false, 0>), dim3(blocks), dim3(GU_WAVES * 64), (uint32_t)lds, st,
                              k_start, k_stop, 0, a, groups, xin, gather_src, act);
    }
    return check_launch("gate_up_mfma");
}

int launch_down_mfma(const ferrite_moe_shape& s, const uint8_t* packed, const ActPlanes& act, int n,
                     const UnitTables& units, void* y, int y_dtype, hipStream_t st) {
    MfmaArgs a = make_args(s, packed, n, units, true);
    const bool x2 = act.q2 != nullptr;
    if (units.unit_rows_cap >= PF_ROWS_X2) {
        if (units.unit_rows_cap != (x2 ? PF_ROWS_X2 : PF_ROWS)) return FERRITE_ERR_INVALID_ARG;
        const int variant = g_prefill_variant.load(std::memory_order_relaxed);
        const bool bf = y_dtype == FERRITE_DT_BF16;
        uint16_t* yh = static_cast<uint16_t*>(y);
        float* yf = static_cast<float*>(y);
        auto go = [&](auto kernel, int W, size_t lds, auto* yp) -> int {
            const int groups = (s.hidden / 64 + W - 1) / W;
            const unsigned blocks = (unsigned)(((size_t)units.max_units * groups + 7) / 8 * 8);
            kernel<<<blocks, W * 64, lds, st>>>(a, groups, act, yp);
            return check_launch("down_stream");
        };
        if (x2) {
            const size_t rows = (size_t)n * s.topk + (s.shared_inter > 0 ? n : 0);
            if (!planes_within_4g(act.q, act.q2, rows * a.act_ld) || !planes_within_4g(act.s, act.s2, rows * scale_pitch(a.act_ld)))
                return FERRITE_ERR_INVALID_ARG;
            constexpr size_t lds = StCfg<8, 8>::LDS_BYTES;
            return bf ? go(down_stream_kernel<8, 8, 2, uint16_t>, 8, lds, yh) : go(down_stream_kernel<8, 8, 2, float>, 8, lds, yf);
        }
        if (variant == 3) {
            constexpr size_t lds = StCfg<4, 8>::LDS_BYTES;
            return bf ? go(down_stream_kernel<4, 8, 1, uint16_t>, 4, lds, yh) : go(down_stream_kernel<4, 8, 1, float>, 4, lds, yf);
        }
        if (variant == 2) {
            constexpr size_t lds = StCfg<8, 8>::LDS_BYTES;
            return bf ? go(down_stream_kernel<8, 8, 1, uint16_t>, 8, lds, yh) : go(down_stream_kernel<8, 8, 1, float>, 8, lds, yf);
        }
        const int groups = (s.hidden / 64 + PF_ITEMS - 1) / PF_ITEMS;
        const unsigned blocks = (unsigned)(((size_t)units.max_units * groups + 7) / 8 * 8);
        int rc;
        if (bf) {
            if ((rc = LdsLimit<&down_prefill_kernel<uint16_t>>::ensure(PF_LDS_BYTES))) return rc;
            down_prefill_kernel<uint16_t><<<blocks, PF_WAVES * 64, PF_LDS_BYTES, st>>>(a, groups, act.q, act.s, yh);
        } else {
            if ((rc = LdsLimit<&down_prefill_kernel<float>>::ensure(PF_LDS_BYTES))) return rc;
            down_prefill_kernel<float><<<blocks, PF_WAVES * 64, PF_LDS_BYTES, st>>>(a, groups, act.q, act.s, yf);
        }
        return check_launch("down_prefill");
    }
    if (units.unit_rows_cap != 16) return FERRITE_ERR_INVALID_ARG;
    const size_t lds = x2 ? b_lds_bytes<true, kWindowKt>(a.act_ld / 128) : b_lds_bytes<false, 0>(a.act_ld / 128);
    const int items = s.hidden / 64;
    const int groups = (items + DN_WAVES * DN_IPW - 1) / (DN_WAVES * DN_IPW);
    const unsigned blocks = (unsigned)(((size_t)units.max_units * groups + 7) / 8 * 8);
    if (y_dtype != FERRITE_DT_F32) return FERRITE_ERR_INVALID_ARG;
    int rc;
    if (x2) {
        if ((rc = LdsLimit<&down_mfma_kernel<DN_WAVES, DN_IPW, true>>::ensure(lds))) return rc;
        down_mfma_kernel<DN_WAVES, DN_IPW, true><<<blocks, DN_WAVES * 64, lds, st>>>(a, groups, act, static_cast<float*>(y));
    } else {
        if ((rc = LdsLimit<&down_mfma_kernel<DN_WAVES, DN_IPW, false>>::ensure(lds))) return rc;
        down_mfma_kernel<DN_WAVES, DN_IPW, false><<<blocks, DN_WAVES * 64, lds, st>>>(a, groups, act, static_cast<float*>(y));
    }
    return check_launch("down_mfma");
}

int warmup_experts_mfma() {
    int rc;
    if ((rc = LdsLimit<&gate_up_mfma_kernel<GU_WAVES, false, 0>>::ensure(kLdsCap))) return rc;
    if ((rc = LdsLimit<&gate_up_mfma_kernel<GU_WAVES, true, kWindowKt>>::ensure(kLdsCap))) return rc;
    if ((rc = LdsLimit<&gate_up_mfma_kernel<GU_WAVES_RESIDENT_X2, true, 0>>::ensure(kLdsCap))) return rc;
    if ((rc = LdsLimit<&down_mfma_kernel<DN_WAVES, DN_IPW, false>>::ensure(kLdsCap))) return rc;
    if ((rc = LdsLimit<&down_mfma_kernel<DN_WAVES, DN_IPW, true>>::ensure(kLdsCap))) return rc;
    if ((rc = LdsLimit<&gate_up_stream_kernel<8, 8, 1>>::ensure(StCfg<8, 8>::LDS_BYTES))) return rc;
    if ((rc = LdsLimit<&gate_up_stream_kernel<8, 8, 2>>::ensure(StCfg<8, 8>::LDS_BYTES))) return rc;
    if ((rc = LdsLimit<&gate_up_prefill_kernel>::ensure(PF_LDS_BYTES))) return rc;
    if ((rc = LdsLimit<&down_prefill_kernel<uint16_t>>::ensure(PF_LDS_BYTES))) return rc;
    return LdsLimit<&down_prefill_kernel<float>>::ensure(PF_LDS_BYTES);
}

}  // namespace fe

using namespace fe;

static int check_shape_mfma(const ferrite_moe_shape* s) {
    if (!s) return FERRITE_ERR_INVALID_ARG;
    if (s->hidden <= 0 || s->inter <= 0 || s->n_experts <= 0 || s->shared_inter < 0) return FERRITE_ERR_INVALID_ARG;
    if (s->hidden % 128 || s->inter % 128 || s->shared_inter % 128) return FERRITE_DECLINED;
    return FERRITE_OK;
}

extern "C" size_t ferrite_moe_packed_bytes(const ferrite_moe_shape* shape) {
    if (check_shape_mfma(shape)) return 0;
    return packed_layout(*shape).total;
}

static int pack_one(const PackSrc& src, int n_experts, uint8_t* codes_dst, uint8_t* scales_dst, hipStream_t st) {
    if (src.rows == 0 || n_experts == 0) return FERRITE_OK;
    const size_t KT = src.K / 128, KT4 = (KT + 3) / 4, items = src.rows / src.rpi;
    size_t nc = items * KT * 256 * n_experts;
    pack_codes_kernel<<<(unsigned)((nc + 255) / 256), 256, 0, st>>>(src, n_experts, reinterpret_cast<uint4*>(codes_dst));
    int rc = check_launch("pack_codes");
    if (rc) return rc;
    size_t ns = items * KT4 * 256 * n_experts;
    pack_scales_kernel<<<(unsigned)((ns + 255) / 256), 256, 0, st>>>(src, n_experts, reinterpret_cast<uint32_t*>(scales_dst));
    return check_launch("pack_scales");
}

extern "C" int ferrite_moe_pack_weights(const ferrite_moe_shape* shape, const ferrite_moe_weights* w, uint8_t* packed,
                                        ferrite_stream_t stream) {
    int rc = check_shape_mfma(shape);
    if (rc) return rc;
    if (!w || !packed || !w->router_w || !w->gate_w || !w->gate_s || !w->up_w || !w->up_s || !w->down_w || !w->down_s)
        return FERRITE_ERR_INVALID_ARG;
    if (shape->shared_inter > 0 && (!w->sh_gate_w || !w->sh_gate_s || !w->sh_up_w || !w->sh_up_s || !w->sh_down_w || !w->sh_down_s))
        return FERRITE_ERR_INVALID_ARG;
    const ferrite_moe_shape& s = *shape;
    PackedLayout L = packed_layout(s);
    hipStream_t st = as_stream(stream);
    if ((rc = launch_router_transpose(w->router_w, s.n_experts, s.hidden, reinterpret_cast<float*>(packed + L.router_t), st)))
        return rc;
    PackSrc gu{{w->gate_w, w->up_w}, {w->gate_s, w->up_s}, s.inter, s.hidden, 2, 32, (size_t)s.hidden / 32};
    if ((rc = pack_one(gu, s.n_experts, packed + L.gu_codes, packed + L.gu_scales, st))) return rc;
    PackSrc dn{{w->down_w, nullptr}, {w->down_s, nullptr}, s.hidden, s.inter, 1, 64, (size_t)s.inter / 32};
    if ((rc = pack_one(dn, s.n_experts, packed + L.dn_codes, packed + L.dn_scales, st))) return rc;
    if (s.shared_inter > 0) {
        PackSrc sgu{{w->sh_gate_w, w->sh_up_w}, {w->sh_gate_s, w->sh_up_s}, s.shared_inter, s.hidden, 2, 32,
                    (size_t)s.hidden / 32};
        if ((rc = pack_one(sgu, 1, packed + L.sh_gu_codes, packed + L.sh_gu_scales, st))) return rc;
        PackSrc sdn{{w->sh_down_w, nullptr}, {w->sh_down_s, nullptr}, s.hidden, s.shared_inter, 1, 64,
                    (size_t)s.shared_inter / 32};
        if ((rc = pack_one(sdn, 1, packed + L.sh_dn_codes, packed + L.sh_dn_scales, st))) return rc;
    }
    return FERRITE_OK;
}

// One expert at a time, for a loader that streams a checkpoint: the same kernels on a single expert's matrices,
// written at that expert's place in the packed buffer.
extern "C" int ferrite_moe_pack_expert(const ferrite_moe_shape* shape, int expert, const ferrite_moe_expert_src* src,
                                       uint8_t* packed, ferrite_stream_t stream) {
    int rc = check_shape_mfma(shape);
    if (rc) return rc;
    const ferrite_moe_shape& s = *shape;
    if (!src || !packed || expert < 0 || expert > s.n_experts) return FERRITE_ERR_INVALID_ARG;
    const bool shared = expert == s.n_experts;
    if (shared && s.shared_inter == 0) return FERRITE_ERR_INVALID_ARG;
    const bool has_gu = src->gate_w || src->gate_s || src->up_w || src->up_s;
    const bool has_dn = src->down_w || src->down_s;
    if (!has_gu && !has_dn) return FERRITE_ERR_INVALID_ARG;
    if (has_gu && (!src->gate_w || !src->gate_s || !src->up_w || !src->up_s)) return FERRITE_ERR_INVALID_ARG;
    if (has_dn && (!src->down_w || !src->down_s)) return FERRITE_ERR_INVALID_ARG;
    const int inter = shared ? s.shared_inter : s.inter;
    const size_t gu_pitch = src->gate_up_scale_pitch ? (size_t)src->gate_up_scale_pitch : (size_t)s.hidden / 32;
    const size_t dn_pitch = src->down_scale_pitch ? (size_t)src->down_scale_pitch : (size_t)inter / 32;
    if (src->gate_up_scale_pitch < 0 || src->down_scale_pitch < 0 || gu_pitch < (size_t)s.hidden / 32 ||
        dn_pitch < (size_t)inter / 32)
        return FERRITE_ERR_INVALID_ARG;
    auto misaligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) != 0; };
    if (misaligned(src->gate_w) || misaligned(src->up_w) || misaligned(src->down_w) || misaligned(packed))
        return FERRITE_DECLINED;
    PackedLayout L = packed_layout(s);
    hipStream_t st = as_stream(stream);
    auto kt4 = [](size_t K) { return (K / 128 + 3) / 4; };
    if (has_gu) {
        const size_t cpe = (size_t)inter * s.hidden, spe = (size_t)(inter / 32) * kt4(s.hidden) * 1024;
        PackSrc gu{{src->gate_w, src->up_w}, {src->gate_s, src->up_s}, inter, s.hidden, 2, 32, gu_pitch};
        uint8_t* cd = packed + (shared ? L.sh_gu_codes : L.gu_codes + (size_t)expert * cpe);
        uint8_t* sd = packed + (shared ? L.sh_gu_scales : L.gu_scales + (size_t)expert * spe);
        if ((rc = pack_one(gu, 1, cd, sd, st))) return rc;
    }
    if (has_dn) {
        const size_t cpe = (size_t)s.hidden * inter / 2, spe = (size_t)(s.hidden / 64) * kt4(inter) * 1024;
        PackSrc dn{{src->down_w, nullptr}, {src->down_s, nullptr}, s.hidden, inter, 1, 64, dn_pitch};
        uint8_t* cd = packed + (shared ? L.sh_dn_codes : L.dn_codes + (size_t)expert * cpe);
        uint8_t* sd = packed + (shared ? L.sh_dn_scales : L.dn_scales + (size_t)expert * spe);
        if ((rc = pack_one(dn, 1, cd, sd, st))) return rc;
    }
    return FERRITE_OK;
}

extern "C" int ferrite_moe_pack_router(const ferrite_moe_shape* shape, const float* router_w, uint8_t* packed,
                                       ferrite_stream_t stream) {
    int rc = check_shape_mfma(shape);
    if (rc) return rc;
    if (!router_w || !packed) return FERRITE_ERR_INVALID_ARG;
    PackedLayout L = packed_layout(*shape);
    return launch_router_transpose(router_w, shape->n_experts, shape->hidden,
                                   reinterpret_cast<float*>(packed + L.router_t), as_stream(stream));
}

// dequantise one matrix out of the packed buffer (verification of the permutation)
__global__ __launch_bounds__(256) void packed_dequant_kernel(const uint4* __restrict__ codes,
                                                             const uint32_t* __restrict__ scales, int rows, int K,
                                                             int nmat, int rpi, int mat, float* __restrict__ dst) {
    // one thread per (row, 32-column block)
    const int KT = K / 128, KT4 = (KT + 3) / 4;
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)rows * (K / 32)) return;
    int row = (int)(idx / (K / 32)), kb = (int)(idx % (K / 32));
    int kt = kb >> 2, g = kb & 3;
    int item = row / rpi, rin = row % rpi;
    const int tpm = 4 / nmat;
    int tile = mat * tpm + rin / 16, lane = g * 16 + (rin & 15);
    uint4 c = codes[(((size_t)item * KT + kt) * 4 + tile) * 64 + lane];
    uint32_t sw = scales[(((size_t)item * KT4 + (kt >> 2)) * 64 + lane) * 4 + tile];
    float s = fe::ue8m0_decode((sw >> (8 * (kt & 3))) & 0xffu);
    uint32_t words[4] = {c.x, c.y, c.z, c.w};
    float* o = dst + (size_t)row * K + (size_t)kb * 32;
    for (int q = 0; q < 4; ++q)
        for (int b = 0; b < 8; ++b) o[q * 8 + b] = fe::e2m1_decode((words[q] >> (4 * b)) & 15u) * s;
}

extern "C" int ferrite_moe_packed_dequant(const ferrite_moe_shape* shape, const uint8_t* packed, int expert, int which,
                                          float* dst, ferrite_stream_t stream) {
    int rc = check_shape_mfma(shape);
    if (rc) return rc;
    const ferrite_moe_shape& s = *shape;
    if (!packed || !dst || which < 0 || which > 2 || expert < 0 || expert > s.n_experts) return FERRITE_ERR_INVALID_ARG;
    const bool shared = expert == s.n_experts;
    if (shared && s.shared_inter == 0) return FERRITE_ERR_INVALID_ARG;
    PackedLayout L = packed_layout(s);
    const int inter = shared ? s.shared_inter : s.inter;
    const bool down = which == 2;
    const int rows = down ? s.hidden : inter, K = down ? inter : s.hidden;
    const size_t KT = K / 128, KT4 = (KT + 3) / 4;
    const int rpi = down ? 64 : 32, nmat = down ? 1 : 2;
    const size_t items = rows / rpi;
    const size_t cpe = items * KT * 4096, spe = items * KT4 * 1024;
    const uint8_t* cb = packed + (shared ? (down ? L.sh_dn_codes : L.sh_gu_codes)
                                         : (down ? L.dn_codes : L.gu_codes) + (size_t)expert * cpe);
    const uint8_t* sb = packed + (shared ? (down ? L.sh_dn_scales : L.sh_gu_scales)
                                         : (down ? L.dn_scales : L.gu_scales) + (size_t)expert * spe);
    size_t total = (size_t)rows * (K / 32);
    packed_dequant_kernel<<<(unsigned)((total + 255) / 256), 256, 0, as_stream(stream)>>>(
        reinterpret_cast<const uint4*>(cb), reinterpret_cast<const uint32_t*>(sb), rows, K, nmat, rpi, down ? 0 : which, dst);
    return check_launch("packed_dequant");
}
