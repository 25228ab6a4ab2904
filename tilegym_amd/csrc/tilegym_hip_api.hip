// C ABI of libtilegym_hip.so (declared in include/tilegym_hip.h): argument validation on the
// host, schedule selection, kernel launches.  No allocation, no synchronisation, no global
// mutable state apart from two thread-local diagnostics (last error text, last schedule).
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <initializer_list>
#include <mutex>

#include "../../include/tilegym_hip.h"
#include "tg_host.h"

// Scratch memory of tg_fp8_gemm_static_scratch: one copy per device the library is loaded on, held until
// the process ends.  In host code this name is only a handle for hipGetSymbolAddress; the device address
// is looked up once per device (scratch_address below) and that pointer is what kernels receive.
static __device__ __align__(256) unsigned char scratch[TG_STATIC_SCRATCH_BYTES];

namespace {

thread_local char g_err[512] = "";
thread_local int32_t g_last_cfg[TG_CFG_COUNT] = {-1, -1, -1, -1, -1, -1, -1, -1, -1};

int32_t fail(int32_t rc, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return rc;
}

int64_t numel(const tg_tensor* t) {
    int64_t n = 1;
    for (int i = 0; i < t->ndim; ++i) n *= t->shape[i];
    return n;
}

bool contiguous(const tg_tensor* t) {
    int64_t expect = 1;
    for (int i = t->ndim - 1; i >= 0; --i) {
        if (t->shape[i] != 1 && t->strides[i] != expect) return false;
        expect *= t->shape[i];
    }
    return true;
}

int32_t check_tensor(const tg_tensor* t, const char* name, int ndim) {
    if (!t) return fail(TG_ERR_NULL, "%s: null tensor descriptor", name);
    if (t->ndim < 0 || t->ndim > TG_MAX_DIMS) return fail(TG_ERR_INVALID, "%s: ndim %d out of range", name, t->ndim);
    if (ndim >= 0 && t->ndim != ndim) return fail(TG_ERR_INVALID, "%s: expected %d dims, got %d", name, ndim, t->ndim);
    for (int i = 0; i < t->ndim; ++i)
        if (t->shape[i] < 0) return fail(TG_ERR_INVALID, "%s: negative extent", name);
    if (!contiguous(t)) return fail(TG_ERR_INVALID, "%s: must be contiguous", name);
    if (numel(t) > 0 && t->ptr == 0) return fail(TG_ERR_NULL, "%s: null data pointer", name);
    return TG_OK;
}

// f32 / f16 / bf16 tensors (inputs of the quantizers, outputs of the dequantizer and the MoE helpers)
int32_t io_type_of(int32_t dtype) {
    switch (dtype) {
        case TG_F32: return tg::OUT_F32;
        case TG_F16: return tg::OUT_F16;
        case TG_BF16: return tg::OUT_BF16;
        default: return -1;
    }
}
// output types of the GEMM entry points: the above plus e4m3fn (saturating round-to-nearest-even cast in the epilogue)
int32_t out_type_of(int32_t dtype) { return dtype == TG_F8E4M3FN ? (int32_t)tg::OUT_F8 : io_type_of(dtype); }

int64_t elem_size(int32_t dtype) {
    switch (dtype) {
        case TG_F32: case TG_I32: return 4;
        case TG_F16: case TG_BF16: return 2;
        case TG_I64: return 8;
        default: return 1;
    }
}

inline int cfg_get(const int32_t* cfg, int32_t ncfg, int slot) {
    return (cfg && slot < ncfg) ? cfg[slot] : -1;
}
inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline bool aligned16(uint64_t p) { return (p & 15) == 0; }

constexpr int64_t kOffsetLimit = (int64_t)1 << 31;  // kernels index operands with 32-bit byte offsets
constexpr int kTargetWaves = 4096;                  // 16 waves on each of 256 CUs
// ragged GEMM: up to this many rows in all take the streaming form (config 5's weights, 64 experts: 6 rows 11.9 / 7.1 us
// against 16.6 / 12.5 for the 64x128 tiles; 24 rows 26.0 / 16.1 against 23.0 / 16.1; 96 rows 60.6 / 35.5 against 59.9 / 32.8)
constexpr int64_t kRaggedStreamRows = 8;
constexpr int64_t kBs256WeightLimit = ((int64_t)1 << 32) - 1;  // the persistent block-scaled kernel addresses all experts' weights with one 32-bit offset

// Switches to the caller's device for the lifetime of a call.
struct DeviceGuard {
    int prev = -1;
    bool ok = false, switched = false;
    explicit DeviceGuard(int dev) {
        int count = 0;
        if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) { (void)hipGetLastError(); return; }
        if (dev < 0 || dev >= count) return;
        if (hipGetDevice(&prev) != hipSuccess) return;
        if (prev != dev) {
            if (hipSetDevice(dev) != hipSuccess) return;
            switched = true;
        }
        ok = true;
    }
    ~DeviceGuard() {
        if (switched) (void)hipSetDevice(prev);
    }
};

// Device address of `scratch` on device `dev`, which must be the current device.  Looked up on the first
// call per device and kept; every device holds its own copy of the array at its own address.
std::mutex g_scratch_mutex;
void* g_scratch_ptr[64] = {nullptr};
hipError_t scratch_address(int dev, uint8_t** out) {
    if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) { (void)hipGetLastError(); return e; }
        if (!ptr) return hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = ptr;
    }
    *out = reinterpret_cast<uint8_t*>(g_scratch_ptr[dev]);
    return hipSuccess;
}

// Bytes of the block scales of a (M, N, K) problem written out per 128 x 128 block, when cfg[] names quantization blocks that are
// larger multiples of 128 (else 0: nothing to write out)
int64_t expanded_scale_bytes(int64_t M, int64_t N, int64_t K, const int32_t* cfg, int32_t ncfg) {
    int64_t qbn = cfg_get(cfg, ncfg, TG_CFG_QUANT_BLOCK_N), qbk = cfg_get(cfg, ncfg, TG_CFG_QUANT_BLOCK_K);
    if (qbn <= 0) qbn = 128;
    if (qbk <= 0) qbk = 128;
    if ((qbn == 128 && qbk == 128) || qbn % 128 != 0 || qbk % 128 != 0) return 0;
    const int64_t kblocks = cdiv(K, 128), nblocks = cdiv(N, 128);
    return (M * kblocks * 4 + 255) / 256 * 256 + (nblocks * kblocks * 4 + 255) / 256 * 256;
}

struct Schedule {
    int kernel;  // 0 fallback, 1 tiled, 2 skinny, 3 stream
    int bm, bn, split_k, row_groups, mt, waves;
};

void remember(const Schedule& s) {
    for (int i = 0; i < TG_CFG_COUNT; ++i) g_last_cfg[i] = -1;
    g_last_cfg[TG_CFG_KERNEL] = s.kernel;
    g_last_cfg[TG_CFG_BLOCK_M] = s.bm;
    g_last_cfg[TG_CFG_BLOCK_N] = s.bn;
    g_last_cfg[TG_CFG_SPLIT_K] = s.split_k;
    g_last_cfg[TG_CFG_ROW_GROUPS] = s.row_groups;
    g_last_cfg[TG_CFG_WAVES] = s.waves;
    g_last_cfg[TG_CFG_PIECES] = 1;
}

// A call that ran as several pieces reports the schedule of its first piece and the number of pieces.
struct PieceRecord {
    int32_t first[TG_CFG_COUNT];
    int count = 0;
    void after_piece() {
        if (count++ == 0) memcpy(first, g_last_cfg, sizeof(first));
    }
    void publish() const {
        if (count == 0) return;
        memcpy(g_last_cfg, first, sizeof(first));
        g_last_cfg[TG_CFG_PIECES] = count;
    }
};

// Tiles of fp8_gemm_tile_mid_kernel.
bool is_mid_tile(int bm, int bn) { return ((bm == 64 || bm == 32) && bn == 32) || (bm == 64 && bn == 64); }

// Per-tensor 64-row tiles of 72 .. 120 weight rows: the deep 64 x 128 kernel with the rest of its weight slab unused.
bool is_narrowed_deep_tile(int bm, int bn) { return bm == 64 && bn >= 72 && bn < 128 && bn % 8 == 0; }

bool tile_exists(int bm, int bn, bool block_scaled) {
    if (is_mid_tile(bm, bn)) return !block_scaled;  // the four waves split K inside the workgroup (per-tensor only)
    if (is_narrowed_deep_tile(bm, bn)) return !block_scaled;
    if (bm == 128 && bn == 128) return true;
    if (bm == 128 && bn == 256) return true;
    if (bm == 64 && bn == 128) return true;
    if (bm == 256 && bn == 256) return true;
    return false;
}

// Split-K factor: `want` if given, else enough to reach `target_units` units of parallel work;
// at least `min_steps` K steps per split, and the partial sums must fit the workspace.
int pick_split(int64_t units, int64_t target_units, int64_t kblocks, int min_steps, int64_t M,
               int64_t N, int64_t partial_bytes_avail, int want) {
    int64_t split = want > 0 ? want : cdiv(target_units, units > 0 ? units : 1);
    if (want <= 0 && split > 16) split = 16;
    const int64_t by_k = kblocks / min_steps > 0 ? kblocks / min_steps : 1;
    if (split > by_k) split = by_k;
    const int64_t per = M * N * 4;
    if (per > 0 && split > 1 && split * per > partial_bytes_avail) split = partial_bytes_avail / per;
    if (split < 1) split = 1;
    // every split must own at least one K step
    const int64_t kps = cdiv(kblocks, split);
    return (int)cdiv(kblocks, kps);
}

// Cost model of the LDS-tiled kernels above 64 rows.  Per tile kind: microseconds per K step of a tile while its compute
// unit holds one workgroup (`alone`: the launch has at most 256 tiles) or two (`shared`), and per tile for set-up, first
// loads and epilogue (`fixed`).  A launch takes rounds x (K steps x step + fixed), rounds = tiles / 256 or tiles / 512
// rounded up, plus, with split-K, the reduction launch (kReduceUs + kReduceUsPerMB x the partial sums).  The numbers are a
// least-squares fit to 9 600 measurements on MI355X: 360 shapes (M = 96 ... 8192, 18 weight shapes, both scalings) x every
// tile x 1 / 2 / 4 / 8 splits, weights rotated past the caches, launches replayed from a graph.  The schedule it picks is
// within 1 % of the best measured one on average (worst case 12 %; the rules it replaces: 7 - 8 % and 2.0 x).
struct TileCost { int bm, bn; float alone, shared, fixed; };
constexpr TileCost kPerTensorTiles[] = {{32, 32, 0.132f, 0.332f, 2.80f},   {64, 32, 0.178f, 0.405f, 3.46f},
                                        {64, 64, 0.249f, 0.596f, 4.43f},   {64, 128, 0.414f, 0.811f, 4.02f},
                                        {128, 128, 0.650f, 0.929f, 3.70f}, {128, 256, 0.874f, 1.782f, 6.88f},
                                        {256, 256, 1.150f, 1.150f, 8.19f}};
// (block-scaled 128 x 256 exists and can be forced; leaving it out of the automatic choice measured better)
constexpr TileCost kBlockScaledTiles[] = {{64, 128, 0.685f, 0.851f, 3.50f}, {128, 128, 0.690f, 1.016f, 4.23f},
                                          {256, 256, 1.496f, 1.496f, 8.11f}};
constexpr float kReduceUs = 6.0f, kReduceUsPerMB = 0.235f;
constexpr float kSplitMargin = 1.05f;  // a split schedule must be predicted this much faster than the best unsplit one

float tile_cost_us(const TileCost& t, int64_t M, int64_t N, int64_t kblocks, int split) {
    const int64_t tiles = cdiv(M, t.bm) * cdiv(N, t.bn) * split, ksteps = cdiv(kblocks, split);
    const bool one_per_cu = t.bm == 256 && t.bn == 256;
    float us = (one_per_cu || tiles <= 256) ? (float)cdiv(tiles, 256) * ((float)ksteps * t.alone + t.fixed)
                                            : (float)cdiv(tiles, 512) * ((float)ksteps * t.shared + t.fixed);
    if (split > 1) us += kReduceUs + kReduceUsPerMB * (float)(M * N * 4 * split) * 1e-6f;
    return us;
}

// The cheapest (tile, split) by the model; a tile (bm > 0) or a split (want_split > 0) given by the caller is kept.
void pick_tile_by_cost(int64_t M, int64_t N, int64_t kblocks, bool block_scaled, int64_t partial_bytes_avail, int want_split,
                       int* bm, int* bn, int* split) {
    const TileCost* kinds = block_scaled ? kBlockScaledTiles : kPerTensorTiles;
    const int n_kinds = block_scaled ? (int)(sizeof(kBlockScaledTiles) / sizeof(TileCost)) : (int)(sizeof(kPerTensorTiles) / sizeof(TileCost));
    float best = 0.f;
    int best_bm = -1, best_bn = -1, best_split = 1;
    for (int i = 0; i < n_kinds; ++i) {
        const TileCost& t = kinds[i];
        if (*bm > 0 && (t.bm != *bm || t.bn != *bn)) continue;
        if (want_split > 1 && is_mid_tile(t.bm, t.bn)) continue;  // these split K inside the workgroup only
        for (int sp = 1; sp <= 8; sp *= 2) {
            if (want_split > 0 && sp != 1) break;          // the caller's split is applied by the caller
            if (sp > 1 && (is_mid_tile(t.bm, t.bn) || kblocks / sp < 4 || (int64_t)sp * M * N * 4 > partial_bytes_avail)) break;
            const float us = tile_cost_us(t, M, N, kblocks, want_split > 0 ? want_split : sp) * (sp > 1 ? kSplitMargin : 1.f);
            if (best_bm < 0 || us < best) { best = us; best_bm = t.bm; best_bn = t.bn; best_split = sp; }
        }
    }
    if (best_bm > 0) { *bm = best_bm; *bn = best_bn; *split = best_split; }
}

// 17 .. 64 rows: the same form of model over more kinds of kernel, with constants of its own (here the weights stream from
// HBM and a tile's step is shorter than above 64 rows; 4 000 measurements, 72 weight x row combinations x both scalings):
// the tile kernels, the wide streaming form (to 32 rows; its "tile" is 64 weight rows x all activation rows, its K step a
// 1 KiB piece) and the skinny kernel (cost proportional to the weight bytes x row tiles, plus a constant).  Against the
// best forced schedule on 72 held-out combinations: 0.4 % (per-tensor) and 0.9 % (block-scaled) behind on average, worst
// 7 % and 16 %; the rules it replaces: 7 % on average, worst 1.4 x and 1.7 x.
struct SmallRowsCosts {
    TileCost tiles[5];
    int n_tiles;
    TileCost wide;                         // bm, bn unused
    float skinny_step, skinny_fixed;       // us per (256 workgroups x K step x row tile), us per launch
    float reduce_us, reduce_us_per_mb;
};
constexpr SmallRowsCosts kSmallPerTensor = {{{32, 32, 0.133f, 0.324f, 3.66f}, {64, 32, 0.167f, 0.426f, 3.98f}, {64, 64, 0.242f, 0.689f, 4.66f},
                                             {64, 128, 0.457f, 1.111f, 3.44f}, {128, 128, 0.714f, 1.192f, 2.38f}}, 5,
                                            {0, 0, 2.446f, 5.599f, 3.54f}, 0.077f, 5.43f, 2.47f, 0.593f};
constexpr SmallRowsCosts kSmallBlockScaled = {{{64, 128, 0.728f, 1.066f, 3.40f}, {128, 128, 0.743f, 1.235f, 3.31f}, {}, {}, {}}, 2,
                                              {0, 0, 3.209f, 6.771f, 3.21f}, 0.102f, 5.42f, 2.47f, 0.549f};

inline float rounds_cost_us(const TileCost& t, int64_t units, int64_t steps) {
    return units <= 256 ? (float)steps * t.alone + t.fixed : (float)cdiv(units, 512) * ((float)steps * t.shared + t.fixed);
}

Schedule choose_dense_tile(int64_t M, int64_t N, int64_t K, bool block_scaled, bool fast_layout,
                           const int32_t* cfg, int32_t ncfg, int64_t partial_bytes_avail);

// The schedule of a dense problem: choose_dense_tile's, and for the per-tensor 64 x 128 tile kernel with fewer workgroups than
// compute units the tile narrowed (120, 112, ... 72 weight rows) as far as the workgroups still fit one round: what a
// workgroup of this weight-streaming regime takes in, (64 + columns) x K bytes, shrinks with it, and more compute units
// take part (28672 x 4096 at M = 64: 224 tiles of 128 columns or 256 of 112).
Schedule choose_dense(int64_t M, int64_t N, int64_t K, bool block_scaled, bool fast_layout,
                      const int32_t* cfg, int32_t ncfg, int64_t partial_bytes_avail) {
    Schedule s = choose_dense_tile(M, N, K, block_scaled, fast_layout, cfg, ncfg, partial_bytes_avail);
    if (s.kernel == 1 && !block_scaled && s.bm == 64 && s.bn == 128 && cfg_get(cfg, ncfg, TG_CFG_BLOCK_N) <= 0) {
        const int64_t tiles_m = cdiv(M, 64);
        if (tiles_m * cdiv(N, 128) * s.split_k < 256) {
            for (int bn = 120; bn >= 72 && tiles_m * cdiv(N, bn) * s.split_k <= 256; bn -= 8) s.bn = bn;
        }
    }
    return s;
}

Schedule choose_dense_tile(int64_t M, int64_t N, int64_t K, bool block_scaled, bool fast_layout,
                           const int32_t* cfg, int32_t ncfg, int64_t partial_bytes_avail) {
    Schedule s{0, -1, -1, 1, -1, -1, -1};
    const int want_kernel = cfg_get(cfg, ncfg, TG_CFG_KERNEL);
    const int64_t kblocks = cdiv(K, 128);
    if (!fast_layout || want_kernel == 0 || K == 0) return s;
    // the block-scaled tiled kernels keep a tile's weight scales for all K steps in LDS (512 steps)
    const bool tile_ok = (K % 128) == 0 && (!block_scaled || kblocks <= 512);
    // above 16 rows the streaming kernels would re-read the activations once per 16 weight rows;
    // the LDS-tiled kernel with a 64-row tile and split-K shares them across 128 weight rows
    bool skinny = M <= 16 || (M <= 64 && !tile_ok);
    if (want_kernel == 1 && tile_ok) skinny = false;
    if ((want_kernel == 2 || want_kernel == 3) && M <= 64) skinny = true;
    // 17 .. 32 rows over a large weight: candidates for the wide streaming form (decided below; otherwise the tile kernels)
    const bool try_wide = !skinny && want_kernel < 0 && M <= 32 && (K % 128) == 0 && N * K >= ((int64_t)48 << 20);
    if (try_wide) skinny = true;
    if (!skinny && !tile_ok) return s;
    const int want_split = cfg_get(cfg, ncfg, TG_CFG_SPLIT_K);
    auto skinny_schedule = [&]() {
        Schedule k{2, -1, -1, 1, -1, -1, -1};
        k.mt = M <= 16 ? 1 : M <= 32 ? 2 : 4;
        int rg = cfg_get(cfg, ncfg, TG_CFG_ROW_GROUPS);
        if (!(rg == 1 || rg == 2 || (rg == 4 && k.mt == 1))) rg = (N >= 16384 && k.mt <= 2) ? 2 : 1;
        k.row_groups = rg;
        const int64_t wgs = cdiv(N, 16 * rg);
        // waves per workgroup: they split K inside the workgroup, no traffic between workgroups
        int nw = cfg_get(cfg, ncfg, TG_CFG_WAVES);
        if (nw != 4 && nw != 8 && nw != 16) {
            nw = wgs * 4 >= kTargetWaves ? 4 : wgs * 8 >= kTargetWaves ? 8 : 16;
            while (nw > 4 && kblocks < nw) nw /= 2;
        }
        k.waves = nw;
        if (want_split > 1 || (want_split < 0 && wgs * nw * 2 <= kTargetWaves))
            k.split_k = pick_split(wgs * nw, kTargetWaves, kblocks, 2 * nw, M, N, partial_bytes_avail, want_split);
        return k;
    };
    // 17 .. 64 rows, nothing but (possibly) the split given by the caller: the cheapest kernel and split by the cost model
    if (want_kernel < 0 && M > 16 && M <= 64 && tile_ok && K >= 1024 && cfg_get(cfg, ncfg, TG_CFG_BLOCK_M) <= 0 &&
        cfg_get(cfg, ncfg, TG_CFG_BLOCK_N) <= 0 && cfg_get(cfg, ncfg, TG_CFG_ROW_GROUPS) < 0 && cfg_get(cfg, ncfg, TG_CFG_WAVES) < 0) {
        const SmallRowsCosts& c = block_scaled ? kSmallBlockScaled : kSmallPerTensor;
        auto reduce = [&](int split) { return split > 1 ? c.reduce_us + c.reduce_us_per_mb * (float)(M * N * 4 * split) * 1e-6f : 0.f; };
        auto fits = [&](int split) { return split == 1 || (int64_t)split * M * N * 4 <= partial_bytes_avail; };
        Schedule best{0, -1, -1, 1, -1, -1, -1};
        float best_us = 0.f;
        auto offer = [&](const Schedule& cand, float us) {
            if (best.kernel == 0 || us < best_us) { best = cand; best_us = us; }  // (no margin against splits here: measured better)
        };
        for (int i = 0; i < c.n_tiles; ++i) {
            const TileCost& t = c.tiles[i];
            const bool mid = is_mid_tile(t.bm, t.bn);
            if (mid && want_split > 1) continue;
            for (int sp = 1; sp <= 8; sp *= 2) {
                const int split = want_split > 0 ? want_split : sp;
                if (split > 1 && (mid || kblocks / split < 4 || !fits(split))) break;
                Schedule cand{1, t.bm, t.bn, 1, -1, -1, -1};
                if (split > 1) cand.split_k = pick_split(cdiv(M, t.bm) * cdiv(N, t.bn), 256, kblocks, 4, M, N, partial_bytes_avail, split);
                offer(cand, rounds_cost_us(t, cdiv(M, t.bm) * cdiv(N, t.bn) * cand.split_k, cdiv(kblocks, cand.split_k)) + reduce(cand.split_k));
                if (want_split > 0) break;
            }
        }
        if (M <= 32) {
            const int64_t pieces = cdiv(K, 1024), wide_wgs = cdiv(N, 64);
            static const int kWideSplits[] = {1, 2, 3, 4, 6, 8};
            for (int sp : kWideSplits) {
                const int split = want_split > 0 ? want_split : sp;
                if (split > pieces || !fits(split)) break;
                Schedule cand{3, -1, -1, 1, 4, 2, 4};
                if (split > 1) cand.split_k = pick_split(wide_wgs, 512, pieces, 1, M, N, partial_bytes_avail, split);
                offer(cand, rounds_cost_us(c.wide, wide_wgs * cand.split_k, cdiv(pieces, cand.split_k)) + reduce(cand.split_k));
                if (want_split > 0) break;
            }
        }
        // (the skinny kernel's time is the least regular of the three; it is the best only for weights of a few MB or
        // very few weight rows, and is offered only there: 2048 x 7168 at M = 32 takes 13.5 us where the model said 9.7)
        if (N * K <= ((int64_t)10 << 20) || N <= 1024) {
            const Schedule cand = skinny_schedule();
            offer(cand, (float)cdiv(N, 16) / 256.f * (float)kblocks * c.skinny_step * (float)cand.mt + c.skinny_fixed + reduce(cand.split_k));
        }
        // the wide form, unsplit: weight rows per workgroup so that the workgroups fill the chip, as for up to 16 rows
        if (best.kernel == 3 && best.row_groups == 4 && best.split_k == 1) {
            int64_t best_cost = 0;
            int rows = 64;
            for (int bn = 64; bn >= 32; bn -= 8) {
                const int64_t cost = cdiv(cdiv(N, bn), 256) * (bn + 16);
                if (bn == 64 || cost < best_cost) { best_cost = cost; rows = bn; }
            }
            if (rows != 64 && cdiv(N, rows) >= 176) best.bn = rows;
        }
        return best;
    }
    const bool nothing_forced = want_kernel < 0 && want_split < 0 && cfg_get(cfg, ncfg, TG_CFG_ROW_GROUPS) < 0 && cfg_get(cfg, ncfg, TG_CFG_WAVES) < 0;
    // up to four rows against a weight of a few MB: the skinny kernel (no LDS, no barrier) is 4 - 19 % ahead of the
    // streaming one (2048 x 2048 block-scaled at M = 1: 4.17 against 4.94 us; per-tensor 4.21 against 4.53)
    if (nothing_forced && M <= 4 && N * K <= ((int64_t)5 << 20)) return skinny_schedule();
    if (skinny && want_kernel != 2 && (want_kernel == 3 || K >= 1024)) {
        // weight streaming through LDS, 1 KiB of a row per load instruction
        s.kernel = 3;
        s.mt = M <= 16 ? 1 : M <= 32 ? 2 : 4;
        s.row_groups = 1;
        s.waves = 4;
        const int64_t pieces = cdiv(K, 1024), wgs = cdiv(N, 16);
        s.split_k = 1;
        // wide variant (64 weight rows per workgroup, activations shared through LDS); ROW_GROUPS = 4 asks for it
        const int want_rg = cfg_get(cfg, ncfg, TG_CFG_ROW_GROUPS);
        const int64_t wide_wgs = cdiv(N, 64);
        // Split-K of the wide form.  A workgroup works through its pieces one memory round trip (~1.5 us) after the other
        // and the reduction launch costs ~3 us: from 136 row blocks on no split pays (12288 x 5120: 12.2 us unsplit, 14.6
        // with two splits; 10240 x 8192: 17.5 against 20.2); below, the workgroups should number about 256, one per
        // compute unit (4096 x 14336, 64 row blocks, M = 1: 22.3 / 16.0 / 13.0 / 14.2 us with 1 / 2 / 4 / 7 splits;
        // 6144 x 8192, 96 row blocks: 14.7 / 12.2 / 12.9 with 1 / 2 / 4) -- counts between one and two per compute unit
        // leave some compute units with twice the work of the others.
        int64_t wide_split = wide_wgs >= 136 ? 1 : 256 / wide_wgs;  // (may be set to 1 below)
        if (wide_split > pieces) wide_split = pieces;
        if (wide_split > 16) wide_split = 16;
        if (wide_wgs >= 112 && pieces < 6) wide_split = 1;  // (8192 x 3072 at M = 16: 7.9 us unsplit, 9.5 with two splits)
        // The wide form wins from 136 row blocks on (11008 x 4096 at M = 16: 11.1 us against 14.3 for the narrow form), and
        // with fewer once the weight is large enough that the reduction launch is paid back: ~32 MB, ~24 MB at more than
        // eight rows where every narrow workgroup's own activation loads weigh more (6144 x 4096 at M = 16: 9.3 against
        // 9.6; 1536 x 24576: 10.4 - 11.9 against 13.5 - 19.4).  One to four rows over 96 - 135 row blocks stay narrow: its
        // 384 - 540 workgroups fill the chip without a reduction (8192 x 8192 at M = 1: 13.6 against 15.7).
        bool wide_auto = N >= 16384 || (wide_wgs >= 136 && K >= 2048) ||
                         (N * K >= ((int64_t)(M > 8 || pieces >= 12 ? 24 : 32) << 20) && wide_wgs * wide_split >= 176 && !(M <= 4 && wide_wgs >= 96));
        // Weight rows per workgroup of the two-piece wide form.  64 rows leave compute units idle when N / 64 is well below 256 or a little above it; fewer rows per
        // workgroup fill the chip in one launch where split-K needed a second one.  Cost of a choice ~ rounds of 256
        // workgroups x (rows + 16): 12288 x 5120 at M = 16 takes 12.6 us with 48 rows (256 workgroups) against 13.2 with
        // 64 (192); 22016 x 4096: 17.3 (48 rows) against 19.9; 8192 x 8192: 13.9 (32 rows, unsplit) against 16.3 (64 rows,
        // two splits); 6144 x 4096: 8.4 (24 rows) against 10.0.  Long K (more than eight 1 KiB pieces) stays with 64 rows
        // and split-K: a workgroup walks its pieces one round trip after the other (4096 x 14336: 14.4 us with four
        // splits, 19.8 unsplit with 24 rows).
        int wide_bn = 64;
        const bool rows_free = (K % 128) == 0 && cfg_get(cfg, ncfg, TG_CFG_BLOCK_N) <= 0 && cfg_get(cfg, ncfg, TG_CFG_WAVES) != 1;
        // (block-scaled: to K = 5120 only -- a piece of its K loop takes longer, and from there on 64 rows with two or
        // more splits win: 8192 x 8192 at M = 16 16.5 us against 19.1 unsplit with 32 rows)
        const int64_t unsplit_pieces = block_scaled ? 5 : 8;
        if (rows_free && M <= 16 && (pieces <= unsplit_pieces || wide_split == 1) && want_split <= 1) {
            int64_t best_cost = 0;
            int best_bn = 64;
            // (long K: 48 rows and more -- 9216 x 16384 takes 25.2 us with 48 rows and 32.5 with 40)
            for (int bn = 64; bn >= (pieces > 8 ? 48 : 24); bn -= 8) {
                const int64_t cost = cdiv(cdiv(N, bn), 256) * (bn + 16);
                if (bn == 64 || cost < best_cost) { best_cost = cost; best_bn = bn; }
            }
            // (too few weight rows to fill the chip even with 24 per workgroup: 64 rows and split-K as before)
            if (cdiv(N, best_bn) >= 176) {
                wide_bn = best_bn;
                if (pieces <= unsplit_pieces) wide_split = 1;
                // with its workgroups filling the chip the wide form also wins at nine rows and more over smaller weights
                // (8192 x 3072 at M = 16: 7.3 against 8.0 us; 5120 x 5120: 9.4 against 11.9)
                if (M > 8 && pieces <= unsplit_pieces) wide_auto = true;
            }
        }
        // long K over one 16-row workgroup per compute unit, one or two activation rows: eight waves split K inside the
        // workgroup, one launch, no partial sums (4096 x 14336: 12.6 us at M = 1 against 13.0 for the wide form with four
        // splits; at M = 8 it is 14.4 against 13.4, and with fewer or more workgroups than compute units it loses by
        // 20 - 35 %: 5120 x 12288, 2048 x 32768)
        const int want_waves = cfg_get(cfg, ncfg, TG_CFG_WAVES);
        // Long K over fewer 16-row workgroups than compute units, the weight too small for the rule above: four waves per
        // workgroup leave the chip idle.  From 112 workgroups on and up to eight rows, eight waves split K inside the workgroup
        // (3072 x 8192 at M = 1: 7.4 us against 8.4; 2048 x 7168: 6.4 against 7.4); else the wide form with up to eight
        // splits (1024 x 16384: 8.3 - 9.1 us against 10.0 - 11.8; 1280 x 8192 at M = 16: 7.7 against 9.1).
        const bool short_of_workgroups = nothing_forced && M <= 16 && !wide_auto && pieces >= 7 && wgs < 224;
        if (short_of_workgroups && wgs >= 112 && M <= 8) {
            s.waves = 8;
            return s;
        }
        if (short_of_workgroups) {
            s.row_groups = 4;
            s.waves = (K % 128) != 0 ? 1 : 4;
            const int64_t want = wide_split < 8 ? wide_split : 8;
            if (want > 1) s.split_k = pick_split(wide_wgs, 512, pieces, 1, M, N, partial_bytes_avail, (int)want);
            return s;
        }
        if (want_rg != 4 && want_split <= 1 && ((want_waves == 8 && M <= 16) || (want_waves < 0 && want_rg < 0 && M <= 2 && pieces >= 8 && wgs >= 224 && wgs <= 256))) {
            s.waves = 8;
            return s;
        }
        // 17 .. 32 rows: the two-piece form with two tiles of activation rows, for weights of 48 MB and more (M = 32,
        // 12288 x 5120 block-scaled: 17.7 us against 24.3 for the 64 x 128 tile kernel with split-K; 4096 x 14336: 16.0
        // against 16.9; 6144 x 4096: 10.6 against 8.4).  Four tiles (to 64 rows) were measured too and lose everywhere
        // (28672 x 4096 at M = 64: 30.4 against 26.3): every wave reads the whole activation piece from LDS.
        const bool wide_rows = M <= 16 || (M <= 32 && (K % 128) == 0);
        if (wide_rows && (want_rg == 4 || (want_rg < 0 && wide_auto && (M <= 16 || N * K >= ((int64_t)48 << 20))))) {
            s.row_groups = 4;
            // K % 128 == 0: the form with two half pieces per wave in flight (reported as WAVES = 4); else, or with
            // WAVES = 1, one 1 KiB piece per wave (reported as WAVES = 1)
            s.waves = (K % 128) != 0 || (want_waves == 1 && M <= 16) ? 1 : 4;
            // weight rows per workgroup of the two-piece form (BLOCK_N = 64, 56, ... 16: 4 x the rows per wave)
            const int want_bn = cfg_get(cfg, ncfg, TG_CFG_BLOCK_N);
            if (s.waves == 4 && want_bn >= 4 && want_bn <= 64 && want_bn % 4 == 0) s.bn = want_bn;
            else if (s.waves == 4 && M <= 16 && wide_bn != 64) s.bn = wide_bn;
            if (want_split > 1) s.split_k = pick_split(wide_wgs, 512, pieces, 1, M, N, partial_bytes_avail, want_split);
            else if (want_split < 0 && wide_split > 1)
                s.split_k = pick_split(wide_wgs, 512, pieces, 1, M, N, partial_bytes_avail, (int)wide_split);
            return s;
        }
        if (!try_wide) {
            if (want_split > 1 || (want_split < 0 && wgs * 4 * 4 <= kTargetWaves && pieces >= 16))
                s.split_k = pick_split(wgs * 4, kTargetWaves / 2, pieces, want_split > 1 ? 1 : 8, M, N, partial_bytes_avail, want_split);
            // weight rows per workgroup of the narrow form (BLOCK_N = 1 .. 16; block-scaled: a divisor of 128)
            const int want_rows = cfg_get(cfg, ncfg, TG_CFG_BLOCK_N);
            if (want_rows >= 1 && want_rows <= 16 && (!block_scaled || 128 % want_rows == 0)) s.bn = want_rows;
            // between one and two workgroups of 16 rows per compute unit, half of the compute units take in twice what the
            // others do; 12 rows per workgroup even that out (6144 x 4096 at M = 8: 8.1 against 8.7 us; 5120 x 5120 at
            // M = 1: 8.9 against 9.5).  More than two per compute unit cost more than they even out (7168 rows: 14 rows
            // per workgroup 6.4 against 6.0 us), and block-scaled workgroups must not straddle a row of weight scales.
            else if (want_rows <= 0 && !block_scaled && s.split_k == 1 && wgs >= 272 && cdiv(N, 12) <= 512) s.bn = 12;
            return s;
        }
        s = Schedule{0, -1, -1, 1, -1, -1, -1};  // not taken by the wide form: on to the tile kernels
        skinny = false;
    }
    if (skinny) return skinny_schedule();
    s.kernel = 1;
    int bm = cfg_get(cfg, ncfg, TG_CFG_BLOCK_M), bn = cfg_get(cfg, ncfg, TG_CFG_BLOCK_N);
    if (!(bm > 0 && bn > 0 && tile_exists(bm, bn, block_scaled))) bm = bn = -1;
    int model_split = 1;
    if (M > 64) {
        pick_tile_by_cost(M, N, kblocks, block_scaled, partial_bytes_avail, want_split, &bm, &bn, &model_split);
    } else if (bm < 0) {
        auto tiles = [&](int64_t a, int64_t b) { return cdiv(M, a) * cdiv(N, b); };
        // small weights at 16 < M <= 64: narrow tiles whose four waves split K inside the workgroup fill the chip in
        // one launch, where the 64x128 tile needs split-K and a reduction launch (4096 x 4096 weight: 7.9 / 7.9 us at
        // M = 32 / 64 against 10.4 / 12.0; 6144 x 4096: 9.4 / 10.2 against 11.8 / 13.3).  Beyond one round of
        // workgroups, or when the weights dominate (>= 32 MiB), the activation re-reads cost more.
        const bool small_w = !block_scaled && N * K <= ((int64_t)32 << 20) && want_split <= 1;
        if (small_w && tiles(32, 32) <= 256) { bm = 32; bn = 32; }
        else if (small_w && tiles(64, 32) <= 256) { bm = 64; bn = 32; }
        else { bm = 64; bn = 128; }
    }
    s.bm = bm;
    s.bn = bn;
    const int64_t wgs = cdiv(M, bm) * cdiv(N, bn);
    s.split_k = 1;
    if (is_mid_tile(bm, bn)) return s;  // K is split inside the workgroup: one launch
    if (want_split > 1) {
        s.split_k = pick_split(wgs, 256, kblocks, 4, M, N, partial_bytes_avail, want_split);
    } else if (M > 64) {
        if (want_split < 0 && model_split > 1) s.split_k = pick_split(wgs, 256, kblocks, 4, M, N, partial_bytes_avail, model_split);
    } else if (want_split < 0 && bm == 64 && bn == 128 && !block_scaled) {
        // weight-streaming regime, four-stage 64x128 kernel (one workgroup per compute unit): the largest
        // power-of-two split that keeps the grid within one round of the chip and >= 8 K steps per split
        // (measured at M = 32 and 64 on the four Llama shapes: 4 / 4 / 1 / 8 for qkv / o / gate+up / down)
        int want = 1;
        while (want < 16 && want * 2 * wgs <= 256 && kblocks / (want * 2) >= 8) want *= 2;
        if (want > 1) s.split_k = pick_split(wgs, want * wgs, kblocks, 4, M, N, partial_bytes_avail, want);
    } else if (want_split < 0 && M <= 64) {
        // weight-streaming regime: at least 128 workgroups and at most 16 K steps per split
        int64_t units = 128;
        if (kblocks / 16 * wgs > units) units = kblocks / 16 * wgs;
        if (units > 512) units = 512;
        int want = 1;
        while (want * wgs < units && want < 16) want *= 2;
        if (want > 1) s.split_k = pick_split(wgs, units, kblocks, 4, M, N, partial_bytes_avail, want);
    }
    return s;
}

struct Resolved {
    int64_t M, N, K;
    bool block_scaled;
    const float* As;
    const float* Bs;
};

// Body of tg_fp8_gemm and tg_fp8_gemm_static_scratch.  static_scratch: the workspace is the library's
// own `scratch` array instead of a caller's buffer, and a problem whose schedule needs more than it holds
// is rejected instead of run with a smaller split.
// piece_ldc: 0 for a whole problem; for a piece of a larger problem (a column or row range computed as a call of its own)
// the row stride of C in elements -- the piece is then described as (M, columns of the piece) and is not split again.
int32_t fp8_gemm_impl(const tg_tensor* c, const tg_tensor* a, const tg_tensor* b, const tg_tensor* scale_a,
                      const tg_tensor* scale_b, int32_t trans_a, int32_t trans_b, float alpha, float beta,
                      const tg_tensor* workspace, bool static_scratch, const int32_t* cfg, int32_t ncfg,
                      int32_t device_id, uint64_t hip_stream, int64_t piece_ldc = 0);

}  // namespace

extern "C" {

int32_t tg_abi_version(void) { return TG_ABI_VERSION; }

const char* tg_rc_message(int32_t rc) {
    switch (rc) {
        case TG_OK: return "ok";
        case TG_ERR_DTYPE: return "unsupported dtype";
        case TG_ERR_LAUNCH: return "kernel launch failed";
        case TG_ERR_DEVICE: return "device init failed";
        case TG_ERR_NULL: return "null tensor pointer";
        case TG_ERR_INVALID: return "invalid arguments";
        default: return "unknown error";
    }
}

const char* tg_last_error(void) { return g_err; }

int32_t tg_last_config(int32_t* out, int32_t n) {
    if (!out || n <= 0) return 0;
    const int32_t m = n < TG_CFG_COUNT ? n : TG_CFG_COUNT;
    for (int32_t i = 0; i < m; ++i) out[i] = g_last_cfg[i];
    return m;
}

// Bytes of the zero-padded operand copies that let a K the MFMA kernels cannot step through run on them anyway: K % 128 != 0
// above 64 rows (the tile kernels take whole 128-byte K blocks), K % 16 != 0 at any row count (the streaming kernels take
// 16-byte pieces).  0 when no padding is needed.
static int64_t padded_k_bytes(int64_t M, int64_t N, int64_t K) {
    if (K <= 0 || (K % 128) == 0 || ((K % 16) == 0 && M <= 64)) return 0;
    const int64_t kp = cdiv(K, 128) * 128;
    return (M * kp + 255) / 256 * 256 + (N * kp + 255) / 256 * 256;
}

int64_t tg_fp8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int32_t trans_b,
                                    const int32_t* cfg, int32_t ncfg) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    int64_t split = cfg_get(cfg, ncfg, TG_CFG_SPLIT_K);
    if (split <= 0) split = 16;
    int64_t bytes = 0;
    // partial sums are only used while they stay a modest part of the traffic
    int64_t partial = split * M * N * 4;
    const int64_t cap = (int64_t)256 << 20;
    if (partial > cap) partial = cap;
    bytes += (partial + 255) / 256 * 256;
    if (!trans_b) bytes += (N * K + 255) / 256 * 256;
    bytes += expanded_scale_bytes(M, N, K, cfg, ncfg);
    bytes += padded_k_bytes(M, N, K);
    return bytes;
}

int32_t tg_fp8_gemm(const tg_tensor* c, const tg_tensor* a, const tg_tensor* b,
                    const tg_tensor* scale_a, const tg_tensor* scale_b, int32_t trans_a,
                    int32_t trans_b, float alpha, float beta, const tg_tensor* workspace,
                    const int32_t* cfg, int32_t ncfg, int32_t device_id, uint64_t hip_stream) {
    // Quantization blocks that are multiples of 128 x 128 (cfg[] slots QUANT_BLOCK_N / _K: 256 x 128, 128 x 256, 256 x 256,
    // ...): the scales are written out per 128 x 128 block at the tail of the workspace (one small launch each) and the
    // problem runs on the MFMA kernels like any 128 x 128 one -- the same products times the same scales, added in the
    // same order.  Without a workspace that holds them, and for finer blocks, the fallback kernel takes the problem.
    // A K that is no multiple of 128 (above 64 rows) or of 16 (any row count): both operands are copied into the tail of the
    // workspace with their rows padded with zeros to the next multiple of 128 -- (K, N) weights are transposed on the way --
    // and the problem runs on the MFMA kernels with the padded K: the same products plus zeros.  Block scales need no
    // change (their last K block was already a partial one).  Without a workspace that holds the copies the fallback
    // kernel takes the problem as before.
    tg_tensor a_pad, b_pad, ws_pad;
    if (a && b && c && workspace && workspace->ptr && a->ptr && b->ptr && a->ndim == 2 && b->ndim == 2 && !trans_a &&
        a->dtype == TG_F8E4M3FN && b->dtype == TG_F8E4M3FN && contiguous(a) && contiguous(b) && cfg_get(cfg, ncfg, TG_CFG_KERNEL) != 0 &&
        // (quantization blocks whose K extent is no multiple of 128 would count another number of blocks over the padded K)
        (cfg_get(cfg, ncfg, TG_CFG_QUANT_BLOCK_K) <= 0 || cfg_get(cfg, ncfg, TG_CFG_QUANT_BLOCK_K) % 128 == 0)) {
        const int64_t M = a->shape[0], K = a->shape[1], N = trans_b ? b->shape[0] : b->shape[1];
        const int64_t need = padded_k_bytes(M, N, K), kp = cdiv(K, 128) * 128;
        const int64_t ws_bytes = numel(workspace) * elem_size(workspace->dtype);
        const bool shapes_ok = (trans_b ? b->shape[1] : b->shape[0]) == K && M > 0 && N > 0 && M <= INT32_MAX && N <= INT32_MAX &&
                               kp <= INT32_MAX && aligned16(workspace->ptr);
        if (need > 0 && shapes_ok && ws_bytes >= need) {
            g_err[0] = 0;
            DeviceGuard guard(device_id);
            if (!guard.ok) return fail(TG_ERR_DEVICE, "cannot use HIP device %d", device_id);
            hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
            uint8_t* tail = reinterpret_cast<uint8_t*>(workspace->ptr) + (ws_bytes - need) / 256 * 256;
            uint8_t* pa = tail;
            uint8_t* pb = tail + (M * kp + 255) / 256 * 256;
            const hipError_t ea = tg::run_pad_rows_u8(reinterpret_cast<const uint8_t*>(a->ptr), pa, (int)M, (int)K, (int)kp, stream);
            const hipError_t eb = trans_b ? tg::run_pad_rows_u8(reinterpret_cast<const uint8_t*>(b->ptr), pb, (int)N, (int)K, (int)kp, stream)
                                          : tg::run_transpose_u8(reinterpret_cast<const uint8_t*>(b->ptr), pb, (int)K, (int)N, (int)kp, stream);
            if (ea != hipSuccess || eb != hipSuccess) return fail(TG_ERR_LAUNCH, "operand padding launch failed");
            a_pad = *a; a_pad.ptr = reinterpret_cast<uint64_t>(pa); a_pad.shape[1] = kp; a_pad.strides[0] = kp; a_pad.strides[1] = 1;
            b_pad = *b; b_pad.ptr = reinterpret_cast<uint64_t>(pb); b_pad.shape[0] = N; b_pad.shape[1] = kp; b_pad.strides[0] = kp; b_pad.strides[1] = 1;
            ws_pad = *workspace; ws_pad.ndim = 1; ws_pad.strides[0] = 1;
            ws_pad.shape[0] = (int64_t)(tail - reinterpret_cast<uint8_t*>(workspace->ptr)) / elem_size(workspace->dtype);
            a = &a_pad; b = &b_pad; workspace = &ws_pad; trans_b = 1;
        }
    }
    const int64_t qbn = cfg_get(cfg, ncfg, TG_CFG_QUANT_BLOCK_N), qbk = cfg_get(cfg, ncfg, TG_CFG_QUANT_BLOCK_K);
    if (a && b && c && scale_a && scale_b && workspace && a->ndim == 2 && b->ndim == 2 && !trans_a && trans_b &&
        cfg_get(cfg, ncfg, TG_CFG_KERNEL) != 0) {
        const int64_t M = a->shape[0], K = a->shape[1], N = b->shape[0];
        const int64_t need = expanded_scale_bytes(M, N, K, cfg, ncfg);
        const int64_t bn = qbn > 0 ? qbn : 128, bk = qbk > 0 ? qbk : 128;
        const int64_t kblocks = cdiv(K, 128), nblocks = cdiv(N, 128), in_cols = cdiv(K, bk);
        const int64_t ws_bytes = workspace->ptr ? numel(workspace) * elem_size(workspace->dtype) : 0;
        const bool shapes_ok = scale_a->dtype == TG_F32 && scale_b->dtype == TG_F32 && scale_a->ndim == 2 && scale_b->ndim == 2 &&
                               scale_a->shape[0] == M && scale_a->shape[1] == in_cols && scale_b->shape[0] == cdiv(N, bn) &&
                               scale_b->shape[1] == in_cols && contiguous(scale_a) && contiguous(scale_b) && scale_a->ptr && scale_b->ptr;
        if (need > 0 && shapes_ok && ws_bytes >= need && M > 0 && N > 0 && K > 0 && M <= INT32_MAX && N <= INT32_MAX && K <= INT32_MAX) {
            g_err[0] = 0;
            DeviceGuard guard(device_id);
            if (!guard.ok) return fail(TG_ERR_DEVICE, "cannot use HIP device %d", device_id);
            hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
            const int64_t a_bytes = (M * kblocks * 4 + 255) / 256 * 256;
            uint8_t* tail = reinterpret_cast<uint8_t*>(workspace->ptr) + (ws_bytes - need) / 256 * 256;
            float* ea = reinterpret_cast<float*>(tail);
            float* eb = reinterpret_cast<float*>(tail + a_bytes);
            if (tg::run_expand_scales(reinterpret_cast<const float*>(scale_a->ptr), ea, (int)M, (int)kblocks, (int)in_cols, 1, (int)(bk / 128), stream) != hipSuccess ||
                tg::run_expand_scales(reinterpret_cast<const float*>(scale_b->ptr), eb, (int)nblocks, (int)kblocks, (int)in_cols, (int)(bn / 128), (int)(bk / 128), stream) != hipSuccess)
                return fail(TG_ERR_LAUNCH, "scale expansion launch failed");
            tg_tensor sa2 = *scale_a, sb2 = *scale_b, ws2 = *workspace;
            sa2.ptr = reinterpret_cast<uint64_t>(ea); sa2.shape[1] = kblocks; sa2.strides[0] = kblocks;
            sb2.ptr = reinterpret_cast<uint64_t>(eb); sb2.shape[0] = nblocks; sb2.shape[1] = kblocks; sb2.strides[0] = kblocks;
            ws2.ndim = 1; ws2.shape[0] = (int64_t)(tail - reinterpret_cast<uint8_t*>(workspace->ptr)) / elem_size(workspace->dtype); ws2.strides[0] = 1;
            int32_t cfg2[TG_CFG_COUNT];
            for (int i = 0; i < TG_CFG_COUNT; ++i) cfg2[i] = cfg_get(cfg, ncfg, i);
            cfg2[TG_CFG_QUANT_BLOCK_N] = cfg2[TG_CFG_QUANT_BLOCK_K] = -1;
            const int32_t rc = fp8_gemm_impl(c, a, b, &sa2, &sb2, trans_a, trans_b, alpha, beta, &ws2, false, cfg2, TG_CFG_COUNT, device_id, hip_stream);
            g_last_cfg[TG_CFG_QUANT_BLOCK_N] = (int32_t)bn;
            g_last_cfg[TG_CFG_QUANT_BLOCK_K] = (int32_t)bk;
            return rc;
        }
    }
    return fp8_gemm_impl(c, a, b, scale_a, scale_b, trans_a, trans_b, alpha, beta, workspace, false, cfg, ncfg,
                         device_id, hip_stream);
}

int32_t tg_fp8_gemm_static_scratch(const tg_tensor* c, const tg_tensor* a, const tg_tensor* b,
                                   const tg_tensor* scale_a, const tg_tensor* scale_b, int32_t trans_a,
                                   int32_t trans_b, float alpha, float beta, const int32_t* cfg, int32_t ncfg,
                                   int32_t device_id, uint64_t hip_stream) {
    return fp8_gemm_impl(c, a, b, scale_a, scale_b, trans_a, trans_b, alpha, beta, nullptr, true, cfg, ncfg,
                         device_id, hip_stream);
}

}  // extern "C"

namespace {

int32_t fp8_gemm_impl(const tg_tensor* c, const tg_tensor* a, const tg_tensor* b, const tg_tensor* scale_a,
                      const tg_tensor* scale_b, int32_t trans_a, int32_t trans_b, float alpha, float beta,
                      const tg_tensor* workspace, bool static_scratch, const int32_t* cfg, int32_t ncfg,
                      int32_t device_id, uint64_t hip_stream, int64_t piece_ldc) {
    g_err[0] = 0;
    int32_t rc;
    const int64_t chunk_ldc = piece_ldc;
    if ((rc = check_tensor(a, "a", 2)) || (rc = check_tensor(b, "b", 2)) || (rc = check_tensor(c, "c", 2))) return rc;
    if (a->dtype != TG_F8E4M3FN || b->dtype != TG_F8E4M3FN)
        return fail(TG_ERR_DTYPE, "a and b must be float8_e4m3fn (dtype code 7), got %d and %d", a->dtype, b->dtype);
    const int out_type = out_type_of(c->dtype);
    if (out_type < 0) return fail(TG_ERR_DTYPE, "c must be bf16, f16, f32 or float8_e4m3fn, got dtype code %d", c->dtype);
    const int64_t M = trans_a ? a->shape[1] : a->shape[0], K = trans_a ? a->shape[0] : a->shape[1];
    const int64_t N = trans_b ? b->shape[0] : b->shape[1], Kb = trans_b ? b->shape[1] : b->shape[0];
    if (K != Kb) return fail(TG_ERR_INVALID, "incompatible matrices: K of a is %lld, K of b is %lld", (long long)K, (long long)Kb);
    if (c->shape[0] != M || c->shape[1] != N)
        return fail(TG_ERR_INVALID, "c must be (%lld, %lld), got (%lld, %lld)", (long long)M, (long long)N, (long long)c->shape[0], (long long)c->shape[1]);
    if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return fail(TG_ERR_INVALID, "extent exceeds int32");
    const int64_t kblocks = cdiv(K, 128), nblocks = cdiv(N, 128);
    const int64_t ldc = chunk_ldc ? chunk_ldc : N;
    // quantization blocks: 128 weight rows x 128 K elements unless cfg[] says otherwise
    int64_t qbn = cfg_get(cfg, ncfg, TG_CFG_QUANT_BLOCK_N), qbk = cfg_get(cfg, ncfg, TG_CFG_QUANT_BLOCK_K);
    if (qbn <= 0) qbn = 128;
    if (qbk <= 0) qbk = 128;
    const bool std_blocks = qbn == 128 && qbk == 128;
    const int64_t sk_cols = cdiv(K, qbk), sb_rows = cdiv(N, qbn);

    // ---- scales (blocks other than 128 x 128 are taken by the fallback kernel only)
    enum Kind { NONE, TENSOR, BLOCK };
    auto kind_of = [&](const tg_tensor* s, const char* name, int64_t rows, int32_t* err) -> Kind {
        *err = TG_OK;
        if (!s) return NONE;
        if ((*err = check_tensor(s, name, -1))) return NONE;
        if (s->dtype != TG_F32) { *err = fail(TG_ERR_DTYPE, "%s must be f32", name); return NONE; }
        if (numel(s) == 1) return TENSOR;
        if (s->ndim == 2 && s->shape[0] == rows && s->shape[1] == sk_cols) return BLOCK;
        *err = fail(TG_ERR_INVALID, "%s: expected 1 element or shape (%lld, %lld)", name, (long long)rows, (long long)sk_cols);
        return NONE;
    };
    const Kind ka = kind_of(scale_a, "scale_a", M, &rc);
    if (rc) return rc;
    const Kind kb = kind_of(scale_b, "scale_b", sb_rows, &rc);
    if (rc) return rc;
    const bool block_scaled = (ka == BLOCK || kb == BLOCK);
    if (block_scaled && (ka == TENSOR || kb == TENSOR) && !(M == 1 && sk_cols == 1) && !(sb_rows == 1 && sk_cols == 1))
        return fail(TG_ERR_INVALID, "scale_a and scale_b must both be per-tensor or both be block scales");
    if (block_scaled && (trans_a || !trans_b))
        return fail(TG_ERR_INVALID, "block scales require a (M,K) and b (N,K) (trans_a=0, trans_b=1)");
    if (workspace) {
        if ((rc = check_tensor(workspace, "workspace", -1))) return rc;
        if (!aligned16(workspace->ptr)) return fail(TG_ERR_INVALID, "workspace must be 16-byte aligned");
    }
    if (M == 0 || N == 0) return TG_OK;

    // ---- column chunks.  The columns of C (rows of an (N, K) weight) can be computed in pieces, each a call of its own on
    // the same stream and workspace; the pieces take C's real row stride as an argument.
    auto run_columns = [&](int64_t n0, int64_t cn, const int32_t* piece_cfg, int32_t piece_ncfg) -> int32_t {
        tg_tensor bs = *b, cs = *c, sbs;
        bs.ptr = b->ptr + (uint64_t)(n0 * K);
        bs.shape[0] = cn;
        cs.ptr = c->ptr + (uint64_t)(n0 * elem_size(c->dtype));
        cs.shape[1] = cn;
        cs.strides[0] = cn;  // described as contiguous; the real row stride is the piece_ldc argument
        const tg_tensor* sb = scale_b;
        if (kb == BLOCK) {
            sbs = *scale_b;
            sbs.ptr = scale_b->ptr + (uint64_t)((n0 / 128) * kblocks * 4);
            sbs.shape[0] = cdiv(cn, 128);
            sb = &sbs;
        }
        return fp8_gemm_impl(&cs, a, &bs, scale_a, sb, trans_a, trans_b, alpha, beta, workspace, static_scratch, piece_cfg, piece_ncfg, device_id, hip_stream, N);
    };
    const bool can_chunk = !chunk_ldc && std_blocks && trans_b && !trans_a && K > 0 && (K % 16) == 0 && aligned16(a->ptr) &&
                           aligned16(b->ptr) && cfg_get(cfg, ncfg, TG_CFG_KERNEL) != 0;
    // (1) weights of 2 GiB and more: the kernels index an operand with 32-bit byte offsets
    if (can_chunk && N * K >= kOffsetLimit && 256 * K < kOffsetLimit) {
        const int64_t chunk_n = ((kOffsetLimit - 1) / K) / 256 * 256;
        PieceRecord pieces;
        for (int64_t n0 = 0; n0 < N; n0 += chunk_n) {
            if ((rc = run_columns(n0, (N - n0) < chunk_n ? (N - n0) : chunk_n, cfg, ncfg))) return rc;
            pieces.after_piece();
        }
        pieces.publish();
        return TG_OK;
    }
    // (2) 256 x 256 tiles whose count leaves the last round of the chip mostly empty (4096 x 5120: 320 tiles, 1.25 rounds):
    // the columns (or rows) that fill whole rounds run with 256 x 256 tiles, the rest as a problem of its own (measured on
    // M = 4096, N = 5120, K = 12288: 206 -> 184 us per-tensor, 251 -> 229 us block-scaled, against 128 x 128 tiles for all).
    if (can_chunk && (K % 128) == 0 && M >= 1024 && cfg_get(cfg, ncfg, TG_CFG_BLOCK_M) <= 0 && cfg_get(cfg, ncfg, TG_CFG_BLOCK_N) <= 0 &&
        cfg_get(cfg, ncfg, TG_CFG_SPLIT_K) <= 0) {
        const int64_t tm = cdiv(M, 256), tn = cdiv(N, 256), total = tm * tn, rounds = cdiv(total, 256);
        if (total > 256 && total * 100 < rounds * 256 * 80) {
            auto fills = [](int64_t tiles) { return tiles >= 256 && tiles * 100 >= cdiv(tiles, 256) * 256 * 95; };
            const int64_t n1 = ((total / 256) * 256) / tm;   // column tiles that fit the whole rounds
            const int64_t m1 = ((total / 256) * 256) / tn;   // or row tiles
            PieceRecord pieces;
            // the piece that fills whole rounds runs with 256 x 256 tiles whatever the cost model would say of it alone
            int32_t full_cfg[TG_CFG_COUNT];
            for (int i = 0; i < TG_CFG_COUNT; ++i) full_cfg[i] = cfg_get(cfg, ncfg, i);
            full_cfg[TG_CFG_KERNEL] = 1;
            full_cfg[TG_CFG_BLOCK_M] = full_cfg[TG_CFG_BLOCK_N] = 256;
            full_cfg[TG_CFG_SPLIT_K] = 1;
            if (n1 >= 1 && n1 < tn && fills(tm * n1)) {
                if ((rc = run_columns(0, n1 * 256, full_cfg, TG_CFG_COUNT))) return rc;
                pieces.after_piece();
                if ((rc = run_columns(n1 * 256, N - n1 * 256, cfg, ncfg))) return rc;
                pieces.after_piece();
                pieces.publish();
                return TG_OK;
            }
            if (m1 >= 1 && m1 < tm && fills(m1 * tn)) {
                // the same along the rows: the pieces are contiguous row ranges of A, C and the activation scales
                for (int piece = 0; piece < 2; ++piece) {
                    const int64_t r0 = piece ? m1 * 256 : 0, rows = piece ? M - m1 * 256 : m1 * 256;
                    tg_tensor as = *a, cs = *c, sas;
                    as.ptr = a->ptr + (uint64_t)(r0 * K);
                    as.shape[0] = rows;
                    cs.ptr = c->ptr + (uint64_t)(r0 * N * elem_size(c->dtype));
                    cs.shape[0] = rows;
                    const tg_tensor* sa = scale_a;
                    if (ka == BLOCK) {
                        sas = *scale_a;
                        sas.ptr = scale_a->ptr + (uint64_t)(r0 * kblocks * 4);
                        sas.shape[0] = rows;
                        sa = &sas;
                    }
                    // (piece_ldc = N marks the call as a piece: no further splitting)
                    rc = fp8_gemm_impl(&cs, &as, b, sa, scale_b, trans_a, trans_b, alpha, beta, workspace, static_scratch,
                                       piece ? cfg : full_cfg, piece ? ncfg : TG_CFG_COUNT, device_id, hip_stream, N);
                    if (rc) return rc;
                    pieces.after_piece();
                }
                pieces.publish();
                return TG_OK;
            }
        }
    }

    DeviceGuard guard(device_id);
    if (!guard.ok) return fail(TG_ERR_DEVICE, "cannot use HIP device %d", device_id);
    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);

    // ---- workspace carving: [split-K partial sums ...][optional K-contiguous copy of B]
    int64_t ws_bytes = workspace ? numel(workspace) * elem_size(workspace->dtype) : 0;
    uint8_t* ws = workspace ? reinterpret_cast<uint8_t*>(workspace->ptr) : nullptr;
    if (static_scratch) {
        const hipError_t e = scratch_address(device_id, &ws);
        if (e != hipSuccess) return fail(TG_ERR_DEVICE, "cannot locate the static scratch buffer on device %d: %s", device_id, hipGetErrorString(e));
        ws_bytes = TG_STATIC_SCRATCH_BYTES;
        const int64_t copy_bytes = (!trans_b && !trans_a && cfg_get(cfg, ncfg, TG_CFG_KERNEL) != 0) ? (N * K + 255) / 256 * 256 : 0;
        if (copy_bytes > ws_bytes)
            return fail(TG_ERR_INVALID, "the K-contiguous copy of a (K,N) weight needs %lld bytes, the static scratch buffer holds %lld: "
                        "pass b as (N,K) with trans_b=1 or call tg_fp8_gemm with a workspace", (long long)copy_bytes, (long long)ws_bytes);
    }
    int64_t ws_free = ws_bytes;
    uint8_t* ws_cursor = ws;

    const uint8_t* Bnt = reinterpret_cast<const uint8_t*>(b->ptr);
    bool b_is_nk = trans_b != 0;
    const int want_kernel = cfg_get(cfg, ncfg, TG_CFG_KERNEL);
    if (!b_is_nk && !trans_a && want_kernel != 0 && K > 0) {
        // (K,N) weights: make a K-contiguous copy at the tail of the workspace when it fits
        const int64_t need = (N * K + 255) / 256 * 256;
        if (ws_free >= need) {
            uint8_t* bt = ws + ws_bytes - need;
            bt = reinterpret_cast<uint8_t*>(reinterpret_cast<uintptr_t>(bt) & ~(uintptr_t)15);
            if (bt >= ws_cursor) {
                if (tg::run_transpose_u8(Bnt, bt, (int)K, (int)N, (int)K, stream) != hipSuccess)
                    return fail(TG_ERR_LAUNCH, "transpose launch failed");
                Bnt = bt;
                b_is_nk = true;
                ws_free = bt - ws_cursor;
            }
        }
    }

    const bool fast_layout = !trans_a && b_is_nk && (K % 16) == 0 && aligned16(a->ptr) &&
                             aligned16(reinterpret_cast<uint64_t>(Bnt)) && N * K < kOffsetLimit && (!block_scaled || std_blocks);
    Schedule s = choose_dense(M, N, K, block_scaled, fast_layout, cfg, ncfg, ws_free);
    if (static_scratch) {
        // same schedule as tg_fp8_gemm with a full-size workspace, or an error: never a silently smaller split
        const Schedule full = choose_dense(M, N, K, block_scaled, fast_layout, cfg, ncfg, INT64_MAX / 2);
        if (full.split_k != s.split_k)
            return fail(TG_ERR_INVALID, "split-K %d of this problem needs %lld bytes of partial sums, the static scratch buffer has %lld free: "
                        "call tg_fp8_gemm with a workspace, or force a smaller SPLIT_K", full.split_k,
                        (long long)full.split_k * M * N * 4, (long long)ws_free);
    }

    tg::GemmParams p{};
    p.A = reinterpret_cast<const uint8_t*>(a->ptr);
    p.B = Bnt;
    p.C = reinterpret_cast<void*>(c->ptr);
    p.As = scale_a ? reinterpret_cast<const float*>(scale_a->ptr) : nullptr;
    p.Bs = scale_b ? reinterpret_cast<const float*>(scale_b->ptr) : nullptr;
    p.M = (int)M; p.N = (int)N; p.K = (int)K;
    p.ldc = (int)ldc;
    p.kblocks = (int)kblocks; p.nblocks = (int)nblocks;
    p.alpha = alpha; p.beta = beta;
    p.out_type = out_type;
    p.vec_store = ((N % 4) == 0 && aligned16(c->ptr) && (ldc == N || (ldc * elem_size(c->dtype)) % 16 == 0)) ? 1 : 0;
    p.split_k = 1;
    p.ksteps_per_split = (int)kblocks;
    p.E = 1; p.top_k = 1;

    if (s.kernel == 0) {
        tg::GenericParams q{};
        q.g = p;
        q.a_sm = trans_a ? 1 : K; q.a_sk = trans_a ? M : 1;
        const bool nk = trans_b != 0;  // the fallback reads the caller's own B
        q.g.B = reinterpret_cast<const uint8_t*>(b->ptr);
        q.b_sn = nk ? K : 1; q.b_sk = nk ? 1 : N;
        q.b_se = 0;
        q.group = tg::GROUP_DENSE;
        q.block_scaled = block_scaled ? 1 : 0;
        q.qbn = (int)qbn; q.qbk = (int)qbk;
        q.rows = (int)M;
        remember(s);
        if (tg::run_generic(q, stream) != hipSuccess) return fail(TG_ERR_LAUNCH, "fallback kernel launch failed");
        return TG_OK;
    }

    if (s.split_k > 1) {
        p.split_k = s.split_k;
        p.ksteps_per_split = (int)cdiv(kblocks, s.split_k);
        p.partials = reinterpret_cast<float*>(ws_cursor);
    }
    remember(s);

    if (s.kernel == 3) {
        const int64_t pieces = cdiv(K, 1024);
        if (s.split_k > 1) p.ksteps_per_split = (int)cdiv(pieces, s.split_k);
        const int64_t per_wave = cdiv(s.split_k > 1 ? p.ksteps_per_split : pieces, 4);
        int nbuf = cfg_get(cfg, ncfg, TG_CFG_ROW_GROUPS);  // stream kernel: LDS buffers per wave
        // measured: one 16 KiB buffer per wave and two workgroups per compute unit beat two buffers and
        // one workgroup, except for long K where they tie
        if (nbuf != 1 && nbuf != 2) nbuf = (per_wave >= 3 && s.mt == 1 && !block_scaled) ? 2 : 1;
        if (s.mt != 1 || s.waves == 8) nbuf = 1;
        if (s.row_groups == 4 && s.waves == 4 && s.bn > 0) p.wave_rows = s.bn / 4;
        if (s.row_groups != 4 && s.bn > 0) p.wave_rows = s.bn;  // narrow form: weight rows per workgroup
        hipError_t e = s.row_groups == 4 ? tg::run_stream_wide(block_scaled, p, s.split_k, stream, s.waves == 4, s.mt)
                                         : tg::run_stream(s.mt, nbuf, s.waves, block_scaled, p, (int)cdiv(N, p.wave_rows > 0 ? p.wave_rows : 16), s.split_k, stream);
        if (e != hipSuccess) return fail(TG_ERR_LAUNCH, "stream kernel launch failed: %s", hipGetErrorString(e));
        if (s.split_k > 1 && tg::run_splitk_reduce(p, block_scaled, stream) != hipSuccess)
            return fail(TG_ERR_LAUNCH, "split-K reduction launch failed");
        return TG_OK;
    }
    if (s.kernel == 2) {
        const int gx = (int)cdiv(N, 16 * s.row_groups);
        hipError_t e = tg::run_skinny(s.mt, s.row_groups, s.waves, block_scaled, p, gx, s.split_k, stream);
        if (e != hipSuccess) return fail(TG_ERR_LAUNCH, "skinny kernel launch failed: %s", hipGetErrorString(e));
        if (s.split_k > 1 && tg::run_splitk_reduce(p, block_scaled, stream) != hipSuccess)
            return fail(TG_ERR_LAUNCH, "split-K reduction launch failed");
        return TG_OK;
    }

    // tiled kernel; rows are chunked so that 32-bit byte offsets into A suffice
    const int64_t max_rows = K > 0 ? ((kOffsetLimit - 1) / K) / s.bm * s.bm : M;
    if (max_rows <= 0) return fail(TG_ERR_INVALID, "K too large");
    for (int64_t r0 = 0; r0 < M; r0 += max_rows) {
        const int64_t rows = (M - r0) < max_rows ? (M - r0) : max_rows;
        tg::GemmParams pc = p;
        pc.A = p.A + r0 * K;
        pc.C = reinterpret_cast<uint8_t*>(p.C) + r0 * ldc * elem_size(c->dtype);  // (ldc, not N: this call may be a column piece of a wider C)
        if (block_scaled && p.As) pc.As = p.As + r0 * kblocks;
        pc.M = (int)rows;
        if (rows != M && s.split_k > 1) { pc.split_k = 1; pc.ksteps_per_split = (int)kblocks; }
        int gx = (int)(cdiv(rows, s.bm) * cdiv(N, s.bn));
        const bool split = pc.split_k > 1;
        const bool deep = s.kernel == 1 && !block_scaled && s.bm == 64 && (s.bn == 128 || is_narrowed_deep_tile(s.bm, s.bn));
        if (deep) pc.tile_cols = s.bn;
        const bool mid = s.kernel == 1 && !block_scaled && is_mid_tile(s.bm, s.bn);
        // persistent kernel with the hand-ordered K loop for the dense per-tensor 256x256 tile, from two K steps up
        // (WAVES = 8 asks for the generic eight-wave tile kernel instead)
        const bool ordered = s.kernel == 1 && !block_scaled && !split && s.bm == 256 && s.bn == 256 && kblocks >= 2 &&
                             cfg_get(cfg, ncfg, TG_CFG_WAVES) != 8;
        // block-scaled 256x256: ROW_GROUPS = 1 asks for the persistent form with three weight slabs (same results; measured
        // within 2 % of the kernel of one workgroup per tile on the dense shapes either way, so it is not the default here)
        const bool bs_persistent = s.kernel == 1 && block_scaled && !split && s.bm == 256 && s.bn == 256 && tg::bs256_takes_k((int)kblocks) &&
                                   N * K < kBs256WeightLimit && pc.As && pc.Bs && cfg_get(cfg, ncfg, TG_CFG_ROW_GROUPS) == 1 &&
                                   cfg_get(cfg, ncfg, TG_CFG_WAVES) != 8;
        if (bs_persistent) g_last_cfg[TG_CFG_ROW_GROUPS] = 1;
        hipError_t e = mid ? tg::run_tile_mid(s.bm, s.bn, pc, stream)
                     : ordered ? tg::run_tile256(pc, gx, stream)
                     : bs_persistent ? tg::run_bs256(tg::GROUP_DENSE, pc, gx, stream)
                     : deep ? tg::run_tile_deep(split, pc, gx, pc.split_k, stream)
                     : block_scaled ? tg::run_tile_block_dense(s.bm, s.bn, split, pc, gx, pc.split_k, stream)
                                    : tg::run_tile_per_tensor(s.bm, s.bn, split, pc, gx, pc.split_k, stream);
        if (e != hipSuccess) return fail(TG_ERR_LAUNCH, "tiled kernel launch failed: %s", hipGetErrorString(e));
        if (split && tg::run_splitk_reduce(pc, block_scaled, stream) != hipSuccess)
            return fail(TG_ERR_LAUNCH, "split-K reduction launch failed");
    }
    return TG_OK;
}

}  // namespace

extern "C" {

// Shared validation of the two grouped entry points.
static int32_t grouped_common(const tg_tensor* c, const tg_tensor* a, const tg_tensor* b,
                              const tg_tensor* a_scale, const tg_tensor* b_scale, int64_t* rows_a,
                              int64_t* E, int64_t* N, int64_t* K, int* out_type, int64_t qbn = 128, int64_t qbk = 128) {
    int32_t rc;
    if ((rc = check_tensor(a, "a", 2)) || (rc = check_tensor(b, "b", 3)) || (rc = check_tensor(c, "c", 2))) return rc;
    if (a->dtype != TG_F8E4M3FN || b->dtype != TG_F8E4M3FN)
        return fail(TG_ERR_DTYPE, "a and b must be float8_e4m3fn (dtype code 7)");
    *out_type = out_type_of(c->dtype);
    if (*out_type < 0) return fail(TG_ERR_DTYPE, "c must be bf16, f16, f32 or float8_e4m3fn");
    *rows_a = a->shape[0];
    *K = a->shape[1];
    *E = b->shape[0];
    *N = b->shape[1];
    if (b->shape[2] != *K) return fail(TG_ERR_INVALID, "K dimensions must match: %lld != %lld", (long long)*K, (long long)b->shape[2]);
    if (c->shape[1] != *N) return fail(TG_ERR_INVALID, "c must have %lld columns", (long long)*N);
    if (*rows_a > INT32_MAX || *N > INT32_MAX || *K > INT32_MAX || *E > INT32_MAX) return fail(TG_ERR_INVALID, "extent exceeds int32");
    const int64_t kblocks = cdiv(*K, qbk), nblocks = cdiv(*N, qbn);  // quantization blocks (128 x 128 unless the caller says otherwise)
    if (a_scale) {
        if ((rc = check_tensor(a_scale, "a_scale", 2))) return rc;
        if (a_scale->dtype != TG_F32) return fail(TG_ERR_DTYPE, "a_scale must be f32");
        if (a_scale->shape[0] != *rows_a || a_scale->shape[1] != kblocks)
            return fail(TG_ERR_INVALID, "a_scale must be (%lld, %lld)", (long long)*rows_a, (long long)kblocks);
    }
    if (b_scale) {
        if ((rc = check_tensor(b_scale, "b_scale", 3))) return rc;
        if (b_scale->dtype != TG_F32) return fail(TG_ERR_DTYPE, "b_scale must be f32");
        if (b_scale->shape[0] != *E || b_scale->shape[1] != nblocks || b_scale->shape[2] != kblocks)
            return fail(TG_ERR_INVALID, "b_scale must be (%lld, %lld, %lld)", (long long)*E, (long long)nblocks, (long long)kblocks);
    }
    return TG_OK;
}

static void fill_grouped(tg::GemmParams& p, const tg_tensor* c, const tg_tensor* a,
                         const tg_tensor* b, const tg_tensor* a_scale, const tg_tensor* b_scale,
                         int64_t rows_c, int64_t E, int64_t N, int64_t K, int out_type) {
    p.A = reinterpret_cast<const uint8_t*>(a->ptr);
    p.B = reinterpret_cast<const uint8_t*>(b->ptr);
    p.C = reinterpret_cast<void*>(c->ptr);
    p.As = a_scale ? reinterpret_cast<const float*>(a_scale->ptr) : nullptr;
    p.Bs = b_scale ? reinterpret_cast<const float*>(b_scale->ptr) : nullptr;
    p.M = (int)rows_c; p.N = (int)N; p.K = (int)K; p.ldc = (int)N;
    p.kblocks = (int)cdiv(K, 128); p.nblocks = (int)cdiv(N, 128);
    p.alpha = 1.0f; p.beta = 0.0f;
    p.out_type = out_type;
    p.vec_store = ((N % 4) == 0 && aligned16(c->ptr)) ? 1 : 0;
    p.split_k = 1;
    p.ksteps_per_split = p.kblocks;
    p.E = (int)E;
    p.top_k = 1;
}

int32_t tg_fp8_ragged_gemm(const tg_tensor* c, const tg_tensor* a, const tg_tensor* b,
                           const tg_tensor* a_scale, const tg_tensor* b_scale,
                           const tg_tensor* m_indptr, const int32_t* cfg, int32_t ncfg,
                           int32_t device_id, uint64_t hip_stream) {
    g_err[0] = 0;
    int64_t total_m, E, N, K;
    int out_type;
    // quantization blocks other than 128 x 128 (cfg[] slots) are taken by the fallback kernel
    int64_t qbn = cfg_get(cfg, ncfg, TG_CFG_QUANT_BLOCK_N), qbk = cfg_get(cfg, ncfg, TG_CFG_QUANT_BLOCK_K);
    if (qbn <= 0) qbn = 128;
    if (qbk <= 0) qbk = 128;
    int32_t rc = grouped_common(c, a, b, a_scale, b_scale, &total_m, &E, &N, &K, &out_type, qbn, qbk);
    if (rc) return rc;
    if (c->shape[0] != total_m) return fail(TG_ERR_INVALID, "c must have %lld rows", (long long)total_m);
    if ((rc = check_tensor(m_indptr, "m_indptr", 1))) return rc;
    if (m_indptr->dtype != TG_I32) return fail(TG_ERR_DTYPE, "m_indptr must be int32");
    if (m_indptr->shape[0] != E + 1) return fail(TG_ERR_INVALID, "m_indptr must have Q+1 = %lld elements", (long long)(E + 1));
    if (total_m == 0 || N == 0 || E == 0) return TG_OK;

    DeviceGuard guard(device_id);
    if (!guard.ok) return fail(TG_ERR_DEVICE, "cannot use HIP device %d", device_id);
    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);

    tg::GemmParams p{};
    fill_grouped(p, c, a, b, a_scale, b_scale, total_m, E, N, K, out_type);
    p.m_indptr = reinterpret_cast<const int*>(m_indptr->ptr);

    const bool fast = (K % 128) == 0 && K > 0 && K <= 65536 && aligned16(a->ptr) && aligned16(b->ptr) &&
                      total_m * K < kOffsetLimit && N * K < kOffsetLimit && qbn == 128 && qbk == 128 &&
                      cfg_get(cfg, ncfg, TG_CFG_KERNEL) != 0;
    Schedule s{0, -1, -1, 1, -1, -1, -1};
    if (!fast) {
        tg::GenericParams q{};
        q.g = p;
        q.a_sm = K; q.a_sk = 1; q.b_sn = K; q.b_sk = 1; q.b_se = N * K;
        q.group = tg::GROUP_RAGGED;
        q.block_scaled = 1;
        q.qbn = (int)qbn; q.qbk = (int)qbk;
        q.rows = (int)total_m;
        remember(s);
        if (tg::run_generic(q, stream) != hipSuccess) return fail(TG_ERR_LAUNCH, "fallback kernel launch failed");
        return TG_OK;
    }
    // One or two tokens' rows over many experts (the batch-1 decode step of a MoE layer): the streaming form, one grid row
    // per expert, reads the weights of the experts that have rows once per 16 rows and nothing of the others.
    // KERNEL = stream asks for it at any row count, KERNEL = tiled for the tile kernels below.
    const int want_kernel = cfg_get(cfg, ncfg, TG_CFG_KERNEL);
    const bool stream_ok = p.As && p.Bs && N * K < ((int64_t)1 << 31) && E <= 65535;
    if (stream_ok && (want_kernel == 3 || (want_kernel < 0 && total_m <= kRaggedStreamRows))) {
        s.kernel = 3; s.row_groups = 4; s.waves = 4;
        // Waves (16 weight rows each) per workgroup: WAVES = 4 / 6 / 8, else the fewest that give the fewest rounds of 256
        // workgroups with rows -- at most one grid row per routed row.  One token of config 5 (six experts): gate+up
        // 264 workgroups of 64 rows 11.5 us, 180 of 96 rows 9.7 us; two tokens, down: 384 of 64 rows 10.8 us, 192 of 128
        // rows 9.3 us; with equal rounds fewer waves are faster (down, one token: 7.0 / 8.4 / 9.0 us for 4 / 6 / 8).
        const int want_waves = cfg_get(cfg, ncfg, TG_CFG_WAVES);
        if (want_waves == 4 || want_waves == 6 || want_waves == 8) {
            s.waves = want_waves;
        } else {
            const int64_t live = total_m < E ? total_m : E;
            int64_t best_rounds = 0;
            for (int w : {4, 6, 8}) {
                const int64_t rounds = cdiv(live * cdiv(N, 16 * w), 256);
                if (w == 4 || rounds < best_rounds) { best_rounds = rounds; s.waves = w; }
            }
        }
        remember(s);
        const hipError_t e = tg::run_stream_ragged(p, s.waves, stream);
        if (e != hipSuccess) return fail(TG_ERR_LAUNCH, "ragged stream kernel launch failed: %s", hipGetErrorString(e));
        return TG_OK;
    }
    int bm = cfg_get(cfg, ncfg, TG_CFG_BLOCK_M), bn = cfg_get(cfg, ncfg, TG_CFG_BLOCK_N);
    if (!(bm > 0 && bn > 0 && tile_exists(bm, bn, true))) {
        // measured on 64 experts of (2816, 2048) weights: padding rows cost no MFMA work (the kernel skips
        // row groups without valid rows), so 256x256 wins from ~96 rows per expert up (101 vs 106-109 us
        // at 96, 172 vs 184-209 at 300), 128x128 down to ~40 (88 vs 102 us at 64), 64x128 below (69 vs 80 at 24)
        if (total_m / E >= 96 && N >= 256) { bm = 256; bn = 256; }
        else { bm = (total_m / E >= 40) ? 128 : 64; bn = 128; }
    }
    s.kernel = 1; s.bm = bm; s.bn = bn;
    remember(s);
    // upper bound on the number of row tiles: every expert adds at most one partial tile
    const int64_t row_tiles = total_m / bm + E;
    const int64_t gx = row_tiles * cdiv(N, bn);
    if (gx > INT32_MAX) return fail(TG_ERR_INVALID, "too many tiles");
    // 256x256: the persistent form (one workgroup per compute unit walks the tiles, the operand rings run on across tiles)
    // hides a tile's set-up and first loads behind the previous tile, which pays for short tiles: measured on 64 experts,
    // 24576 rows, 104 vs 112 us at K = 1408 (11 steps per tile), but 215 vs 196 us at K = 2048 (16 steps), where the
    // hardware's dispatch of one workgroup per tile balances the partly filled row tiles better than a fixed walk.
    // ROW_GROUPS = 1 asks for it, WAVES = 8 for the kernel of one workgroup per tile.
    const int want_form = cfg_get(cfg, ncfg, TG_CFG_ROW_GROUPS);
    const bool persistent = bm == 256 && bn == 256 && p.As && p.Bs && tg::bs256_takes_k(p.kblocks) && E * N * K < kBs256WeightLimit &&
                            cfg_get(cfg, ncfg, TG_CFG_WAVES) != 8 && (want_form == 1 || (want_form < 0 && p.kblocks <= 12));
    if (persistent) g_last_cfg[TG_CFG_ROW_GROUPS] = 1;
    hipError_t e = persistent ? tg::run_bs256(tg::GROUP_RAGGED, p, (int)gx, stream)
                              : tg::run_tile_block_grouped(bm, bn, tg::GROUP_RAGGED, p, (int)gx, stream);
    if (e != hipSuccess) return fail(TG_ERR_LAUNCH, "grouped kernel launch failed: %s", hipGetErrorString(e));
    return TG_OK;
}

int32_t tg_fp8_moe_gemm(const tg_tensor* c, const tg_tensor* a, const tg_tensor* b,
                        const tg_tensor* a_scale, const tg_tensor* b_scale,
                        const tg_tensor* topk_weights, const tg_tensor* sorted_token_ids,
                        const tg_tensor* expert_ids, const tg_tensor* num_tokens_post_padded,
                        int32_t mul_routed_weight, int32_t top_k, int32_t block_m,
                        const int32_t* cfg, int32_t ncfg, int32_t device_id, uint64_t hip_stream) {
    g_err[0] = 0;
    int64_t T, E, N, K;
    int out_type;
    int32_t rc = grouped_common(c, a, b, a_scale, b_scale, &T, &E, &N, &K, &out_type);
    if (rc) return rc;
    if (top_k <= 0) return fail(TG_ERR_INVALID, "top_k must be positive");
    if (block_m <= 0 || block_m % 16) return fail(TG_ERR_INVALID, "block_m must be a positive multiple of 16");
    const int64_t num_valid = c->shape[0];
    if (num_valid > T * top_k) return fail(TG_ERR_INVALID, "c has %lld rows but a provides only %lld slots", (long long)num_valid, (long long)(T * top_k));
    if ((rc = check_tensor(sorted_token_ids, "sorted_token_ids", 1)) || (rc = check_tensor(expert_ids, "expert_ids", 1)) ||
        (rc = check_tensor(num_tokens_post_padded, "num_tokens_post_padded", -1)))
        return rc;
    if (sorted_token_ids->dtype != TG_I32 || expert_ids->dtype != TG_I32 || num_tokens_post_padded->dtype != TG_I32)
        return fail(TG_ERR_DTYPE, "sorted_token_ids, expert_ids and num_tokens_post_padded must be int32");
    if (numel(num_tokens_post_padded) < 1) return fail(TG_ERR_INVALID, "num_tokens_post_padded must hold one element");
    const int64_t EM = sorted_token_ids->shape[0];
    if (expert_ids->shape[0] * block_m < EM)
        return fail(TG_ERR_INVALID, "expert_ids too short: %lld blocks of %d for %lld slots", (long long)expert_ids->shape[0], block_m, (long long)EM);
    if (mul_routed_weight) {
        if (!topk_weights) return fail(TG_ERR_NULL, "topk_weights required when mul_routed_weight is set");
        if ((rc = check_tensor(topk_weights, "topk_weights", -1))) return rc;
        if (topk_weights->dtype != TG_F32) return fail(TG_ERR_DTYPE, "topk_weights must be f32");
        if (numel(topk_weights) < num_valid) return fail(TG_ERR_INVALID, "topk_weights too short");
    }
    if (num_valid == 0 || N == 0 || EM == 0) return TG_OK;

    DeviceGuard guard(device_id);
    if (!guard.ok) return fail(TG_ERR_DEVICE, "cannot use HIP device %d", device_id);
    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);

    tg::GemmParams p{};
    fill_grouped(p, c, a, b, a_scale, b_scale, num_valid, E, N, K, out_type);
    p.sorted_ids = reinterpret_cast<const int*>(sorted_token_ids->ptr);
    p.expert_ids = reinterpret_cast<const int*>(expert_ids->ptr);
    p.num_post_pad = reinterpret_cast<const int*>(num_tokens_post_padded->ptr);
    p.row_weight = mul_routed_weight ? reinterpret_cast<const float*>(topk_weights->ptr) : nullptr;
    p.top_k = top_k;
    p.num_valid = (int)num_valid;
    p.block_m = block_m;
    p.em_capacity = (int)EM;

    int bm = cfg_get(cfg, ncfg, TG_CFG_BLOCK_M), bn = cfg_get(cfg, ncfg, TG_CFG_BLOCK_N);
    if (!(bm > 0 && bn > 0 && tile_exists(bm, bn, true) && block_m % bm == 0)) {
        if (block_m % 256 == 0 && N >= 256) { bm = 256; bn = 256; }
        else { bm = (block_m % 128 == 0) ? 128 : (block_m % 64 == 0) ? 64 : 0; bn = 128; }
    }
    const bool fast = bm > 0 && (K % 128) == 0 && K > 0 && K <= 65536 && aligned16(a->ptr) && aligned16(b->ptr) &&
                      T * K < kOffsetLimit && N * K < kOffsetLimit && cfg_get(cfg, ncfg, TG_CFG_KERNEL) != 0;
    Schedule s{0, -1, -1, 1, -1, -1, -1};
    if (!fast) {
        tg::GenericParams q{};
        q.g = p;
        q.a_sm = K; q.a_sk = 1; q.b_sn = K; q.b_sk = 1; q.b_se = N * K;
        q.group = tg::GROUP_GATHER;
        q.block_scaled = 1;
        q.qbn = 128; q.qbk = 128;
        q.rows = (int)EM;
        remember(s);
        if (tg::run_generic(q, stream) != hipSuccess) return fail(TG_ERR_LAUNCH, "fallback kernel launch failed");
        return TG_OK;
    }
    s.kernel = 1; s.bm = bm; s.bn = bn;
    remember(s);
    const int64_t gx = cdiv(EM, bm) * cdiv(N, bn);
    if (gx > INT32_MAX) return fail(TG_ERR_INVALID, "too many tiles");
    hipError_t e = tg::run_tile_block_grouped(bm, bn, tg::GROUP_GATHER, p, (int)gx, stream);
    if (e != hipSuccess) return fail(TG_ERR_LAUNCH, "grouped kernel launch failed: %s", hipGetErrorString(e));
    return TG_OK;
}

int32_t tg_fp8_moe_gemm_silu_quant(const tg_tensor* q, const tg_tensor* scales, const tg_tensor* a, const tg_tensor* b,
                                   const tg_tensor* a_scale, const tg_tensor* b_scale,
                                   const tg_tensor* sorted_token_ids, const tg_tensor* expert_ids,
                                   const tg_tensor* num_tokens_post_padded, int32_t top_k, int32_t block_m,
                                   int32_t act_dtype, int32_t device_id, uint64_t hip_stream) {
    g_err[0] = 0;
    int32_t rc;
    if ((rc = check_tensor(a, "a", 2)) || (rc = check_tensor(b, "b", 3)) || (rc = check_tensor(q, "q", 2)) ||
        (rc = check_tensor(scales, "scales", 2)) || (rc = check_tensor(a_scale, "a_scale", 2)) ||
        (rc = check_tensor(b_scale, "b_scale", 3)) || (rc = check_tensor(sorted_token_ids, "sorted_token_ids", 1)) ||
        (rc = check_tensor(expert_ids, "expert_ids", 1)) || (rc = check_tensor(num_tokens_post_padded, "num_tokens_post_padded", -1)))
        return rc;
    if (a->dtype != TG_F8E4M3FN || b->dtype != TG_F8E4M3FN || q->dtype != TG_F8E4M3FN)
        return fail(TG_ERR_DTYPE, "a, b and q must be float8_e4m3fn (dtype code 7)");
    if (scales->dtype != TG_F32 || a_scale->dtype != TG_F32 || b_scale->dtype != TG_F32)
        return fail(TG_ERR_DTYPE, "scales, a_scale and b_scale must be f32");
    if (act_dtype != TG_BF16 && act_dtype != TG_F16) return fail(TG_ERR_DTYPE, "act_dtype must be bf16 or f16");
    if (sorted_token_ids->dtype != TG_I32 || expert_ids->dtype != TG_I32 || num_tokens_post_padded->dtype != TG_I32)
        return fail(TG_ERR_DTYPE, "sorted_token_ids, expert_ids and num_tokens_post_padded must be int32");
    const int64_t T = a->shape[0], K = a->shape[1], E = b->shape[0], N = b->shape[1], I = N / 2;
    if (b->shape[2] != K) return fail(TG_ERR_INVALID, "K dimensions must match: %lld != %lld", (long long)K, (long long)b->shape[2]);
    if (N % 2 || I % 128 || I == 0) return fail(TG_ERR_INVALID, "b must hold 2*I rows per expert with I a positive multiple of 128 (got %lld)", (long long)N);
    if (K % 128 || K == 0 || K > 65536) return fail(TG_ERR_INVALID, "K must be a multiple of 128 in [128, 65536]");
    if (top_k <= 0) return fail(TG_ERR_INVALID, "top_k must be positive");
    if (block_m <= 0 || block_m % 128) return fail(TG_ERR_INVALID, "block_m must be a positive multiple of 128 for the fused form");
    const int64_t num_valid = q->shape[0];
    if (q->shape[1] != I) return fail(TG_ERR_INVALID, "q must have %lld columns", (long long)I);
    if (num_valid > T * top_k) return fail(TG_ERR_INVALID, "q has %lld rows but a provides only %lld slots", (long long)num_valid, (long long)(T * top_k));
    if (scales->shape[0] != num_valid || scales->shape[1] != I / 128)
        return fail(TG_ERR_INVALID, "scales must be (%lld, %lld)", (long long)num_valid, (long long)(I / 128));
    if (a_scale->shape[0] != T || a_scale->shape[1] != K / 128) return fail(TG_ERR_INVALID, "a_scale must be (%lld, %lld)", (long long)T, (long long)(K / 128));
    if (b_scale->shape[0] != E || b_scale->shape[1] != N / 128 || b_scale->shape[2] != K / 128)
        return fail(TG_ERR_INVALID, "b_scale must be (%lld, %lld, %lld)", (long long)E, (long long)(N / 128), (long long)(K / 128));
    if (!contiguous(q) || !contiguous(scales) || !contiguous(a) || !contiguous(b) || !contiguous(a_scale) || !contiguous(b_scale))
        return fail(TG_ERR_INVALID, "all tensors must be contiguous");
    if (numel(num_tokens_post_padded) < 1) return fail(TG_ERR_INVALID, "num_tokens_post_padded must hold one element");
    const int64_t EM = sorted_token_ids->shape[0];
    if (expert_ids->shape[0] * block_m < EM)
        return fail(TG_ERR_INVALID, "expert_ids too short: %lld blocks of %d for %lld slots", (long long)expert_ids->shape[0], block_m, (long long)EM);
    if (T > INT32_MAX || N > INT32_MAX || E > INT32_MAX || T * K >= kOffsetLimit || N * K >= kOffsetLimit)
        return fail(TG_ERR_INVALID, "extent too large for the fused form");
    if (!aligned16(a->ptr) || !aligned16(b->ptr) || (q->ptr % 8) != 0) return fail(TG_ERR_INVALID, "a and b must be 16-byte aligned, q 8-byte aligned");
    if (num_valid == 0 || EM == 0) return TG_OK;

    DeviceGuard guard(device_id);
    if (!guard.ok) return fail(TG_ERR_DEVICE, "cannot use HIP device %d", device_id);
    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);

    tg::GemmParams p{};
    p.A = reinterpret_cast<const uint8_t*>(a->ptr);
    p.B = reinterpret_cast<const uint8_t*>(b->ptr);
    p.C = reinterpret_cast<void*>(q->ptr);
    p.As = reinterpret_cast<const float*>(a_scale->ptr);
    p.Bs = reinterpret_cast<const float*>(b_scale->ptr);
    p.M = (int)num_valid; p.N = (int)N; p.K = (int)K; p.ldc = (int)N;
    p.kblocks = (int)(K / 128); p.nblocks = (int)(N / 128);
    p.alpha = 1.0f; p.beta = 0.0f;
    p.out_type = act_dtype == TG_BF16 ? tg::OUT_BF16 : tg::OUT_F16;
    p.split_k = 1;
    p.ksteps_per_split = p.kblocks;
    p.E = (int)E;
    p.sorted_ids = reinterpret_cast<const int*>(sorted_token_ids->ptr);
    p.expert_ids = reinterpret_cast<const int*>(expert_ids->ptr);
    p.num_post_pad = reinterpret_cast<const int*>(num_tokens_post_padded->ptr);
    p.top_k = top_k;
    p.num_valid = (int)num_valid;
    p.block_m = block_m;
    p.em_capacity = (int)EM;
    p.inter = (int)I;
    p.act_scales = reinterpret_cast<float*>(scales->ptr);
    p.act_is_bf16 = act_dtype == TG_BF16 ? 1 : 0;

    const int bm = block_m % 256 == 0 ? 256 : 128;  // a row tile must not span two alignment blocks (experts)
    Schedule s{1, bm, 256, 1, -1, -1, -1};
    remember(s);
    const int64_t gx = cdiv(EM, bm) * (I / 128);
    if (gx > INT32_MAX) return fail(TG_ERR_INVALID, "too many tiles");
    hipError_t e = tg::run_tile_moe_act(bm, p, (int)gx, stream);
    if (e != hipSuccess) return fail(TG_ERR_LAUNCH, "fused MoE kernel launch failed: %s", hipGetErrorString(e));
    return TG_OK;
}

// argument checks of moe_align_block_size (host side only); n = number of (token, slot) pairs, cap = len(sorted_token_ids)
static int32_t check_align_args(const tg_tensor* topk_ids, int32_t block_size, int32_t num_experts,
                                const tg_tensor* sorted_token_ids, const tg_tensor* expert_ids,
                                const tg_tensor* num_tokens_post_padded, const tg_tensor* cumsum,
                                const tg_tensor* max_expert_count, int64_t* n_out, int64_t* cap_out) {
    int32_t rc;
    if ((rc = check_tensor(topk_ids, "topk_ids", -1)) || (rc = check_tensor(sorted_token_ids, "sorted_token_ids", 1)) ||
        (rc = check_tensor(expert_ids, "expert_ids", 1)) || (rc = check_tensor(num_tokens_post_padded, "num_tokens_post_padded", -1)) ||
        (rc = check_tensor(cumsum, "cumsum", 1)) || (rc = check_tensor(max_expert_count, "max_expert_count", -1)))
        return rc;
    if (topk_ids->dtype != TG_I32 && topk_ids->dtype != TG_I64) return fail(TG_ERR_DTYPE, "topk_ids must be int32 or int64");
    const tg_tensor* outs[5] = {sorted_token_ids, expert_ids, num_tokens_post_padded, cumsum, max_expert_count};
    for (const tg_tensor* t : outs)
        if (t->dtype != TG_I32) return fail(TG_ERR_DTYPE, "outputs must be int32");
    if (block_size < 1) return fail(TG_ERR_INVALID, "block_size must be positive");
    if (num_experts < 1 || num_experts > 512) return fail(TG_ERR_INVALID, "num_experts must be in [1, 512], got %d", num_experts);
    const int64_t n = numel(topk_ids);
    const int64_t cap = n + (int64_t)num_experts * (block_size - 1);
    if (cap > INT32_MAX) return fail(TG_ERR_INVALID, "too many (token, slot) pairs");
    const int64_t nblk = cdiv(cap, block_size);
    if (numel(sorted_token_ids) != cap) return fail(TG_ERR_INVALID, "sorted_token_ids must have %lld elements", (long long)cap);
    if (numel(expert_ids) < nblk) return fail(TG_ERR_INVALID, "expert_ids must have at least %lld elements", (long long)nblk);
    if (numel(num_tokens_post_padded) < 1 || numel(max_expert_count) < 1) return fail(TG_ERR_INVALID, "scalar outputs need one element");
    if (numel(cumsum) != num_experts + 1) return fail(TG_ERR_INVALID, "cumsum must have num_experts + 1 elements");
    *n_out = n;
    *cap_out = cap;
    return TG_OK;
}

int32_t tg_moe_align_block_size(const tg_tensor* topk_ids, int32_t block_size, int32_t num_experts,
                                const tg_tensor* sorted_token_ids, const tg_tensor* expert_ids,
                                const tg_tensor* num_tokens_post_padded, const tg_tensor* cumsum,
                                const tg_tensor* max_expert_count, int32_t device_id, uint64_t hip_stream) {
    g_err[0] = 0;
    int64_t n, cap;
    const int32_t rc = check_align_args(topk_ids, block_size, num_experts, sorted_token_ids, expert_ids, num_tokens_post_padded, cumsum,
                                        max_expert_count, &n, &cap);
    if (rc) return rc;
    DeviceGuard guard(device_id);
    if (!guard.ok) return fail(TG_ERR_DEVICE, "cannot use HIP device %d", device_id);
    hipError_t e = tg::run_moe_align(reinterpret_cast<const void*>(topk_ids->ptr), topk_ids->dtype == TG_I64, (int)n, num_experts,
                                     block_size, reinterpret_cast<int*>(sorted_token_ids->ptr), (int)cap,
                                     reinterpret_cast<int*>(expert_ids->ptr), (int)numel(expert_ids),
                                     reinterpret_cast<int*>(num_tokens_post_padded->ptr), reinterpret_cast<int*>(cumsum->ptr),
                                     reinterpret_cast<int*>(max_expert_count->ptr), reinterpret_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(TG_ERR_LAUNCH, "moe_align launch failed: %s", hipGetErrorString(e));
    return TG_OK;
}

int32_t tg_moe_align_quant_1x128(const tg_tensor* topk_ids, int32_t block_size, int32_t num_experts,
                                 const tg_tensor* sorted_token_ids, const tg_tensor* expert_ids,
                                 const tg_tensor* num_tokens_post_padded, const tg_tensor* cumsum,
                                 const tg_tensor* max_expert_count, const tg_tensor* q, const tg_tensor* scales,
                                 const tg_tensor* x, int32_t device_id, uint64_t hip_stream) {
    g_err[0] = 0;
    int64_t n, cap;
    int32_t rc = check_align_args(topk_ids, block_size, num_experts, sorted_token_ids, expert_ids, num_tokens_post_padded, cumsum,
                                  max_expert_count, &n, &cap);
    if (rc) return rc;
    if ((rc = check_tensor(x, "x", -1)) || (rc = check_tensor(q, "q", -1)) || (rc = check_tensor(scales, "scales", -1))) return rc;
    if (x->dtype != TG_BF16 && x->dtype != TG_F16) return fail(TG_ERR_DTYPE, "x must be bf16 or f16");
    if (q->dtype != TG_F8E4M3FN) return fail(TG_ERR_DTYPE, "q must be float8_e4m3fn (dtype code 7)");
    if (scales->dtype != TG_F32) return fail(TG_ERR_DTYPE, "scales must be f32");
    if (x->ndim < 1) return fail(TG_ERR_INVALID, "x needs at least one dimension");
    const int64_t K = x->shape[x->ndim - 1], nx = numel(x);
    if (K % 128 != 0) return fail(TG_ERR_INVALID, "the last dimension (%lld) must be a multiple of 128", (long long)K);
    if (numel(q) != nx) return fail(TG_ERR_INVALID, "q must have the shape of x");
    const int64_t groups = nx / 128;
    if (numel(scales) != groups) return fail(TG_ERR_INVALID, "scales must have %lld elements", (long long)groups);
    if (nx > 0 && (!aligned16(x->ptr) || (q->ptr & 7) != 0)) return fail(TG_ERR_INVALID, "x must be 16-byte and q 8-byte aligned");
    DeviceGuard guard(device_id);
    if (!guard.ok) return fail(TG_ERR_DEVICE, "cannot use HIP device %d", device_id);
    hipError_t e = tg::run_moe_align_quant(reinterpret_cast<const void*>(topk_ids->ptr), topk_ids->dtype == TG_I64, (int)n, num_experts,
                                           block_size, reinterpret_cast<int*>(sorted_token_ids->ptr), (int)cap,
                                           reinterpret_cast<int*>(expert_ids->ptr), (int)numel(expert_ids),
                                           reinterpret_cast<int*>(num_tokens_post_padded->ptr), reinterpret_cast<int*>(cumsum->ptr),
                                           reinterpret_cast<int*>(max_expert_count->ptr), reinterpret_cast<const void*>(x->ptr),
                                           x->dtype == TG_BF16, reinterpret_cast<uint8_t*>(q->ptr), reinterpret_cast<float*>(scales->ptr),
                                           groups, reinterpret_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(TG_ERR_LAUNCH, "moe_align + quantizer launch failed: %s", hipGetErrorString(e));
    return TG_OK;
}


int32_t tg_fp8_quant_group(const tg_tensor* q, const tg_tensor* scales, const tg_tensor* x, int32_t group_size,
                           float eps, int32_t rule, int32_t device_id, uint64_t hip_stream) {
    g_err[0] = 0;
    int32_t rc;
    if ((rc = check_tensor(x, "x", -1)) || (rc = check_tensor(q, "q", -1))) return rc;
    if (!scales) return fail(TG_ERR_NULL, "scales: null tensor descriptor");
    if (scales->ndim < 0 || scales->ndim > TG_MAX_DIMS) return fail(TG_ERR_INVALID, "scales: ndim %d out of range", scales->ndim);
    const int x_type = io_type_of(x->dtype);
    if (x_type < 0) return fail(TG_ERR_DTYPE, "x must be bf16, f16 or f32");
    if (q->dtype != TG_F8E4M3FN && q->dtype != TG_I8) return fail(TG_ERR_DTYPE, "q must be float8_e4m3fn (dtype code 7) or int8 (8)");
    if (scales->dtype != TG_F32) return fail(TG_ERR_DTYPE, "scales must be f32");
    if (rule < 0 || rule > 2) return fail(TG_ERR_INVALID, "rule must be 0, 1 or 2");
    if (group_size != 16 && group_size != 32 && group_size != 64 && group_size != 128)
        return fail(TG_ERR_INVALID, "group_size must be 16, 32, 64 or 128, got %d", group_size);
    if (x->ndim < 1) return fail(TG_ERR_INVALID, "x needs at least one dimension");
    const int64_t K = x->shape[x->ndim - 1], n = numel(x);
    if (K % group_size != 0) return fail(TG_ERR_INVALID, "the last dimension (%lld) must be a multiple of %d", (long long)K, group_size);
    if (numel(q) != n) return fail(TG_ERR_INVALID, "q must have the shape of x");
    const int64_t groups = n / group_size, gpr = K / group_size, rows = K > 0 ? n / K : 0;
    if (numel(scales) != groups) return fail(TG_ERR_INVALID, "scales must have %lld elements", (long long)groups);
    bool strided = false;
    int64_t s_row = gpr, s_col = 1;
    if (!contiguous(scales)) {
        if (scales->ndim != 2 || scales->shape[0] != rows || scales->shape[1] != gpr)
            return fail(TG_ERR_INVALID, "strided scales must be 2-D (%lld, %lld)", (long long)rows, (long long)gpr);
        s_row = scales->strides[0], s_col = scales->strides[1];
        if (s_row < 0 || s_col < 0) return fail(TG_ERR_INVALID, "scales: negative stride");
        // two (row, group) pairs must not share an element: one stride has to step over the other dimension
        const bool col_major = s_row >= 1 && s_col >= s_row * rows, row_major = s_col >= 1 && s_row >= s_col * gpr;
        if (groups > 1 && !col_major && !row_major) return fail(TG_ERR_INVALID, "scales: overlapping strides");
        if (groups > INT32_MAX) return fail(TG_ERR_INVALID, "too many groups for strided scales");
        strided = true;
    }
    if (groups > 0 && scales->ptr == 0) return fail(TG_ERR_NULL, "scales: null data pointer");
    if (!aligned16(x->ptr) || (q->ptr & 7) != 0) return fail(TG_ERR_INVALID, "x must be 16-byte and q 8-byte aligned");
    if (n == 0) return TG_OK;
    DeviceGuard guard(device_id);
    if (!guard.ok) return fail(TG_ERR_DEVICE, "cannot use HIP device %d", device_id);
    hipError_t e = tg::run_act_quant_group(reinterpret_cast<const void*>(x->ptr), x_type, reinterpret_cast<uint8_t*>(q->ptr),
                                           q->dtype == TG_I8, reinterpret_cast<float*>(scales->ptr), groups, group_size, eps, rule, strided, gpr,
                                           s_row, s_col, reinterpret_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(TG_ERR_LAUNCH, "quantizer launch failed: %s", hipGetErrorString(e));
    return TG_OK;
}

int32_t tg_fp8_quant_1x128(const tg_tensor* q, const tg_tensor* scales, const tg_tensor* x, float eps,
                           int32_t rule, int32_t device_id, uint64_t hip_stream) {
    g_err[0] = 0;
    int32_t rc;
    if ((rc = check_tensor(x, "x", -1)) || (rc = check_tensor(q, "q", -1)) || (rc = check_tensor(scales, "scales", -1))) return rc;
    if (rule != 0 && rule != 1) return fail(TG_ERR_INVALID, "rule must be 0 or 1");
    return tg_fp8_quant_group(q, scales, x, 128, eps, rule, device_id, hip_stream);
}

int32_t tg_fp8_weight_dequant(const tg_tensor* y, const tg_tensor* x, const tg_tensor* s, int32_t block_size,
                              int32_t device_id, uint64_t hip_stream) {
    g_err[0] = 0;
    int32_t rc;
    if ((rc = check_tensor(x, "x", 2)) || (rc = check_tensor(y, "y", 2)) || (rc = check_tensor(s, "s", 2))) return rc;
    if (x->dtype != TG_F8E4M3FN) return fail(TG_ERR_DTYPE, "x must be float8_e4m3fn (dtype code 7)");
    if (s->dtype != TG_F32) return fail(TG_ERR_DTYPE, "s must be f32");
    const int y_type = io_type_of(y->dtype);
    if (y_type < 0) return fail(TG_ERR_DTYPE, "y must be bf16, f16 or f32");
    if (block_size < 1) return fail(TG_ERR_INVALID, "block_size must be positive");
    const int64_t M = x->shape[0], N = x->shape[1];
    if (y->shape[0] != M || y->shape[1] != N) return fail(TG_ERR_INVALID, "y must be (%lld, %lld)", (long long)M, (long long)N);
    if (s->shape[0] != cdiv(M, block_size) || s->shape[1] != cdiv(N, block_size))
        return fail(TG_ERR_INVALID, "s must be (%lld, %lld)", (long long)cdiv(M, block_size), (long long)cdiv(N, block_size));
    if (M == 0 || N == 0) return TG_OK;
    const bool vec = N % 16 == 0 && block_size % 16 == 0 && aligned16(x->ptr) && aligned16(y->ptr);
    const int64_t work = vec ? M * (N / 16) : M * N;
    if (cdiv(work, 256) > INT32_MAX) return fail(TG_ERR_INVALID, "weight too large");
    DeviceGuard guard(device_id);
    if (!guard.ok) return fail(TG_ERR_DEVICE, "cannot use HIP device %d", device_id);
    hipError_t e = tg::run_weight_dequant(reinterpret_cast<const uint8_t*>(x->ptr), reinterpret_cast<const float*>(s->ptr),
                                          reinterpret_cast<void*>(y->ptr), y_type, M, N, block_size, s->shape[1], vec,
                                          reinterpret_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(TG_ERR_LAUNCH, "dequantizer launch failed: %s", hipGetErrorString(e));
    return TG_OK;
}

int32_t tg_silu_mul_quant_1x128(const tg_tensor* q, const tg_tensor* scales, const tg_tensor* x,
                                int32_t device_id, uint64_t hip_stream) {
    g_err[0] = 0;
    int32_t rc;
    if ((rc = check_tensor(x, "x", 2)) || (rc = check_tensor(q, "q", 2)) || (rc = check_tensor(scales, "scales", 2))) return rc;
    const int x_type = io_type_of(x->dtype);
    if (x_type != tg::OUT_BF16 && x_type != tg::OUT_F16) return fail(TG_ERR_DTYPE, "x must be bf16 or f16");
    if (q->dtype != TG_F8E4M3FN) return fail(TG_ERR_DTYPE, "q must be float8_e4m3fn (dtype code 7)");
    if (scales->dtype != TG_F32) return fail(TG_ERR_DTYPE, "scales must be f32");
    const int64_t R = x->shape[0], I = x->shape[1] / 2;
    if (x->shape[1] % 2 != 0 || I % 8 != 0) return fail(TG_ERR_INVALID, "x must be (R, 2*I) with I a multiple of 8");
    if (I > INT32_MAX / 4) return fail(TG_ERR_INVALID, "row too long");
    if (q->shape[0] != R || q->shape[1] != I) return fail(TG_ERR_INVALID, "q must be (%lld, %lld)", (long long)R, (long long)I);
    if (scales->shape[0] != R || scales->shape[1] != cdiv(I, 128))
        return fail(TG_ERR_INVALID, "scales must be (%lld, %lld)", (long long)R, (long long)cdiv(I, 128));
    if (!aligned16(x->ptr) || (q->ptr & 7) != 0) return fail(TG_ERR_INVALID, "x must be 16-byte and q 8-byte aligned");
    if (R == 0 || I == 0) return TG_OK;
    DeviceGuard guard(device_id);
    if (!guard.ok) return fail(TG_ERR_DEVICE, "cannot use HIP device %d", device_id);
    hipError_t e = tg::run_silu_mul_quant(reinterpret_cast<const void*>(x->ptr), x_type, reinterpret_cast<uint8_t*>(q->ptr),
                                          reinterpret_cast<float*>(scales->ptr), R, (int)I, reinterpret_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(TG_ERR_LAUNCH, "silu_mul_quant launch failed: %s", hipGetErrorString(e));
    return TG_OK;
}

int32_t tg_moe_sum(const tg_tensor* out, const tg_tensor* x, int32_t device_id, uint64_t hip_stream) {
    g_err[0] = 0;
    int32_t rc;
    if ((rc = check_tensor(x, "x", 3)) || (rc = check_tensor(out, "out", 2))) return rc;
    const int x_type = io_type_of(x->dtype);
    if ((x_type != tg::OUT_BF16 && x_type != tg::OUT_F16) || out->dtype != x->dtype)
        return fail(TG_ERR_DTYPE, "x and out must both be bf16 or both f16");
    const int64_t T = x->shape[0], k = x->shape[1], H = x->shape[2];
    if (out->shape[0] != T || out->shape[1] != H) return fail(TG_ERR_INVALID, "out must be (%lld, %lld)", (long long)T, (long long)H);
    if (k < 1 || k > INT32_MAX || H > INT32_MAX || H % 8 != 0) return fail(TG_ERR_INVALID, "top_k must be positive and H a multiple of 8");
    if (!aligned16(x->ptr) || !aligned16(out->ptr)) return fail(TG_ERR_INVALID, "x and out must be 16-byte aligned");
    if (T == 0 || H == 0) return TG_OK;
    DeviceGuard guard(device_id);
    if (!guard.ok) return fail(TG_ERR_DEVICE, "cannot use HIP device %d", device_id);
    hipError_t e = tg::run_moe_sum(reinterpret_cast<const void*>(x->ptr), reinterpret_cast<void*>(out->ptr), x_type, T, (int)k, (int)H,
                                   reinterpret_cast<hipStream_t>(hip_stream));
    if (e != hipSuccess) return fail(TG_ERR_LAUNCH, "moe_sum launch failed: %s", hipGetErrorString(e));
    return TG_OK;
}

int32_t tg_fp8_group_gemm(const tg_tensor* const* c, const tg_tensor* const* a, const tg_tensor* const* b,
                          const tg_tensor* const* scale_a, const tg_tensor* const* scale_b, int32_t count,
                          int32_t trans_b, const tg_tensor* workspace, const int32_t* cfg, int32_t ncfg,
                          int32_t device_id, uint64_t hip_stream) {
    g_err[0] = 0;
    if (count < 0) return fail(TG_ERR_INVALID, "negative count");
    if (count == 0) return TG_OK;
    if (!c || !a || !b) return fail(TG_ERR_NULL, "null descriptor array");
    // ---- can the whole list go out as one launch?
    bool one_launch = trans_b != 0 && cfg_get(cfg, ncfg, TG_CFG_KERNEL) != 0 && cfg_get(cfg, ncfg, TG_CFG_SPLIT_K) <= 1;
    int32_t rc;
    int32_t out_dtype = -1;
    int64_t max_m = 0;
    for (int i = 0; i < count; ++i) {
        if ((rc = check_tensor(a[i], "a[i]", 2)) || (rc = check_tensor(b[i], "b[i]", 2)) || (rc = check_tensor(c[i], "c[i]", 2))) return rc;
        if (a[i]->dtype != TG_F8E4M3FN || b[i]->dtype != TG_F8E4M3FN) return fail(TG_ERR_DTYPE, "a and b must be float8_e4m3fn (dtype code 7)");
        if (out_type_of(c[i]->dtype) < 0) return fail(TG_ERR_DTYPE, "c must be bf16, f16, f32 or float8_e4m3fn");
        if (out_dtype < 0) out_dtype = c[i]->dtype;
        if (c[i]->dtype != out_dtype) one_launch = false;
        const int64_t M = a[i]->shape[0], K = a[i]->shape[1];
        const int64_t N = trans_b ? b[i]->shape[0] : b[i]->shape[1], Kb = trans_b ? b[i]->shape[1] : b[i]->shape[0];
        if (K != Kb) return fail(TG_ERR_INVALID, "problem %d: K dimensions must match: %lld != %lld", i, (long long)K, (long long)Kb);
        if (c[i]->shape[0] != M || c[i]->shape[1] != N) return fail(TG_ERR_INVALID, "problem %d: c must be (%lld, %lld)", i, (long long)M, (long long)N);
        for (const tg_tensor* const* sc : {scale_a, scale_b}) {
            if (sc && sc[i]) {
                if ((rc = check_tensor(sc[i], "scale", -1))) return rc;
                if (sc[i]->dtype != TG_F32 || numel(sc[i]) != 1) return fail(TG_ERR_INVALID, "problem %d: scales must be one-element f32 tensors", i);
            }
        }
        if (K <= 0 || K % 128 != 0 || K > 65536 || !aligned16(a[i]->ptr) || !aligned16(b[i]->ptr) || M * K >= kOffsetLimit ||
            N * K >= kOffsetLimit || M > INT32_MAX || N > INT32_MAX)
            one_launch = false;
        if (M > max_m) max_m = M;
    }
    if (!one_launch) {
        for (int i = 0; i < count; ++i) {
            rc = tg_fp8_gemm(c[i], a[i], b[i], scale_a ? scale_a[i] : nullptr, scale_b ? scale_b[i] : nullptr, 0, trans_b, 1.0f, 0.0f,
                             workspace, cfg, ncfg, device_id, hip_stream);
            if (rc) return rc;
        }
        return TG_OK;
    }
    DeviceGuard guard(device_id);
    if (!guard.ok) return fail(TG_ERR_DEVICE, "cannot use HIP device %d", device_id);
    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
    int bm = cfg_get(cfg, ncfg, TG_CFG_BLOCK_M), bn = cfg_get(cfg, ncfg, TG_CFG_BLOCK_N);
    if (!((bm == 256 && bn == 256) || (bm == 128 && bn == 128) || (bm == 64 && bn == 128))) {
        int64_t big = 0;
        for (int i = 0; i < count; ++i) big += cdiv(a[i]->shape[0], 256) * cdiv(b[i]->shape[0], 256);
        if (max_m <= 64) { bm = 64; bn = 128; }
        else if (big >= 200) { bm = 256; bn = 256; }
        else { bm = 128; bn = 128; }
    }
    Schedule s{1, bm, bn, 1, -1, -1, -1};
    remember(s);
    for (int first = 0; first < count; first += tg::kListMax) {
        tg::GemmList gl{};
        gl.out_type = out_type_of(out_dtype);
        gl.alpha = 1.0f;
        int tiles = 0;
        for (int i = first; i < count && i < first + tg::kListMax; ++i) {
            const int64_t M = a[i]->shape[0], N = b[i]->shape[0], K = a[i]->shape[1];
            if (M == 0 || N == 0) continue;
            tg::ListProblem& q = gl.prob[gl.count++];
            q.A = reinterpret_cast<const uint8_t*>(a[i]->ptr);
            q.B = reinterpret_cast<const uint8_t*>(b[i]->ptr);
            q.C = reinterpret_cast<void*>(c[i]->ptr);
            q.As = (scale_a && scale_a[i]) ? reinterpret_cast<const float*>(scale_a[i]->ptr) : nullptr;
            q.Bs = (scale_b && scale_b[i]) ? reinterpret_cast<const float*>(scale_b[i]->ptr) : nullptr;
            q.M = (int)M; q.N = (int)N; q.K = (int)K;
            tiles += (int)(cdiv(M, bm) * cdiv(N, bn));
            q.tile_end = tiles;
            q.vec_store = ((N % 4) == 0 && aligned16(c[i]->ptr)) ? 1 : 0;
        }
        if (gl.count == 0 || tiles == 0) continue;
        hipError_t e = tg::run_tile_list(bm, bn, gl, tiles, stream);
        if (e != hipSuccess) return fail(TG_ERR_LAUNCH, "list kernel launch failed: %s", hipGetErrorString(e));
    }
    return TG_OK;
}

// ---- the MoE layer as one call: carve the workspace, describe the pieces, run the four entry points above
}  // extern "C"

namespace {
struct MoeLayout {
    int64_t sorted_ids, expert_ids, post, cumsum, max_count, xq, xs, q2, s2, c3, total;  // byte offsets
    int64_t cap, nblk;
};
MoeLayout moe_layout(int64_t T, int64_t k, int64_t E, int64_t H, int64_t I, int64_t block_m, int64_t elem16) {
    MoeLayout l{};
    auto take = [&](int64_t bytes) { const int64_t at = l.total; l.total += (bytes + 255) / 256 * 256; return at; };
    l.cap = T * k + E * (block_m - 1);
    l.nblk = cdiv(l.cap, block_m);
    l.sorted_ids = take(l.cap * 4);
    l.expert_ids = take((l.nblk > 0 ? l.nblk : 1) * 4);
    l.post = take(4);
    l.cumsum = take((E + 1) * 4);
    l.max_count = take(4);
    l.xq = take(T * H);
    l.xs = take(T * (H / 128) * 4);
    l.q2 = take(T * k * I);
    l.s2 = take(T * k * cdiv(I, 128) * 4);
    l.c3 = take(T * k * H * elem16);
    return l;
}
tg_tensor describe(uint8_t* base, int64_t offset, int32_t dtype, std::initializer_list<int64_t> shape) {
    tg_tensor t{};
    t.ptr = reinterpret_cast<uint64_t>(base + offset);
    t.ndim = (int32_t)shape.size();
    int i = 0;
    for (int64_t d : shape) t.shape[i++] = d;
    int64_t stride = 1;
    for (int j = t.ndim - 1; j >= 0; --j) {
        t.strides[j] = stride;
        stride *= t.shape[j];
    }
    t.dtype = dtype;
    return t;
}
}  // namespace

extern "C" {

int64_t tg_fp8_fused_moe_workspace_bytes(int64_t tokens, int64_t top_k, int64_t experts, int64_t hidden, int64_t inter,
                                         int32_t block_m) {
    if (tokens < 0 || top_k < 1 || experts < 1 || hidden < 1 || inter < 1 || block_m < 1) return 0;
    return moe_layout(tokens, top_k, experts, hidden, inter, block_m, 2).total;
}

int32_t tg_fp8_fused_moe(const tg_tensor* out, const tg_tensor* hidden, const tg_tensor* w1, const tg_tensor* w2,
                         const tg_tensor* w1_scale, const tg_tensor* w2_scale, const tg_tensor* topk_weights,
                         const tg_tensor* topk_ids, const tg_tensor* workspace, int32_t block_m, int32_t device_id,
                         uint64_t hip_stream) {
    g_err[0] = 0;
    int32_t rc;
    if ((rc = check_tensor(out, "out", 2)) || (rc = check_tensor(hidden, "hidden", 2)) || (rc = check_tensor(w1, "w1", 3)) ||
        (rc = check_tensor(w2, "w2", 3)) || (rc = check_tensor(w1_scale, "w1_scale", 3)) || (rc = check_tensor(w2_scale, "w2_scale", 3)) ||
        (rc = check_tensor(topk_weights, "topk_weights", 2)) || (rc = check_tensor(topk_ids, "topk_ids", 2)) ||
        (rc = check_tensor(workspace, "workspace", -1)))
        return rc;
    const int act = io_type_of(hidden->dtype);
    if ((act != tg::OUT_BF16 && act != tg::OUT_F16) || out->dtype != hidden->dtype)
        return fail(TG_ERR_DTYPE, "hidden and out must both be bf16 or both f16");
    if (topk_weights->dtype != TG_F32) return fail(TG_ERR_DTYPE, "topk_weights must be f32");
    const int64_t T = hidden->shape[0], H = hidden->shape[1], E = w1->shape[0], I = w1->shape[1] / 2, k = topk_ids->shape[1];
    if (out->shape[0] != T || out->shape[1] != H) return fail(TG_ERR_INVALID, "out must be (%lld, %lld)", (long long)T, (long long)H);
    if (w1->shape[1] != 2 * I || w1->shape[2] != H || w2->shape[0] != E || w2->shape[1] != H || w2->shape[2] != I)
        return fail(TG_ERR_INVALID, "w1 must be (E, 2I, H) and w2 (E, H, I)");
    if (topk_ids->shape[0] != T || topk_weights->shape[0] != T || topk_weights->shape[1] != k || k < 1)
        return fail(TG_ERR_INVALID, "topk_weights and topk_ids must both be (T, k)");
    if (block_m != 128 && block_m != 256) return fail(TG_ERR_INVALID, "block_m must be 128 or 256");
    if ((2 * I) % 256 != 0 || H % 128 != 0) return fail(TG_ERR_INVALID, "this entry point needs 2I %% 256 == 0 and H %% 128 == 0");
    if (T == 0) return TG_OK;
    const int64_t elem16 = 2;
    const MoeLayout l = moe_layout(T, k, E, H, I, block_m, elem16);
    if (l.cap > INT32_MAX) return fail(TG_ERR_INVALID, "too many (token, slot) pairs");
    if (numel(workspace) * elem_size(workspace->dtype) < l.total)
        return fail(TG_ERR_INVALID, "workspace holds %lld bytes, the layer needs %lld", (long long)(numel(workspace) * elem_size(workspace->dtype)),
                    (long long)l.total);
    if (workspace->ptr % 256 != 0) return fail(TG_ERR_INVALID, "workspace must be 256-byte aligned");
    uint8_t* ws = reinterpret_cast<uint8_t*>(workspace->ptr);
    const tg_tensor sorted_ids = describe(ws, l.sorted_ids, TG_I32, {l.cap});
    const tg_tensor expert_ids = describe(ws, l.expert_ids, TG_I32, {l.nblk});
    const tg_tensor post = describe(ws, l.post, TG_I32, {1});
    const tg_tensor cumsum = describe(ws, l.cumsum, TG_I32, {E + 1});
    const tg_tensor max_count = describe(ws, l.max_count, TG_I32, {1});
    const tg_tensor xq = describe(ws, l.xq, TG_F8E4M3FN, {T, H});
    const tg_tensor xs = describe(ws, l.xs, TG_F32, {T, H / 128});
    const tg_tensor q2 = describe(ws, l.q2, TG_F8E4M3FN, {T * k, I});
    const tg_tensor s2 = describe(ws, l.s2, TG_F32, {T * k, cdiv(I, 128)});
    const tg_tensor c3 = describe(ws, l.c3, hidden->dtype, {T, k, H});
    const tg_tensor c3_rows = describe(ws, l.c3, hidden->dtype, {T * k, H});
    const tg_tensor weights_flat = describe(reinterpret_cast<uint8_t*>(topk_weights->ptr), 0, TG_F32, {T * k});
    if ((rc = tg_moe_align_quant_1x128(topk_ids, block_m, (int32_t)E, &sorted_ids, &expert_ids, &post, &cumsum, &max_count, &xq, &xs, hidden,
                                       device_id, hip_stream)))
        return rc;
    if ((rc = tg_fp8_moe_gemm_silu_quant(&q2, &s2, &xq, w1, &xs, w1_scale, &sorted_ids, &expert_ids, &post, (int32_t)k, block_m, hidden->dtype,
                                         device_id, hip_stream)))
        return rc;
    if ((rc = tg_fp8_moe_gemm(&c3_rows, &q2, w2, &s2, w2_scale, &weights_flat, &sorted_ids, &expert_ids, &post, 1, 1, block_m, nullptr, 0,
                              device_id, hip_stream)))
        return rc;
    return tg_moe_sum(out, &c3, device_id, hip_stream);
}

}  // extern "C"
