// extern "C" entry points of libkiln_marlin_gemm (device side) and the
// dispatcher that replaces `marlin_cuda` (crates/kiln-marlin-gemm/csrc/marlin_kernel.cu:731-819).
#include <initializer_list>
#include <mutex>
#include <unordered_map>

#include "kiln_w4a16.h"
#include "device_common.h"
#include "launch.h"

namespace kiln {

namespace {

constexpr int kMaxDevices = 16;
// The workspace prefix that is zero between launches (launch.h): counters and the sticky word of the
// bounded waits, then the region in which K slices exchange partial tiles without counters, whose end
// holds the flags and counts of a LoRA projection folded into its GEMM's launch.
constexpr size_t kCounterBytes = kWsCounterBytes;
constexpr size_t kCounterCapacity = kWsCounterCapacity;  // what counters may use of it
constexpr size_t kFlaggedBytes = kWsFlaggedBytes;
constexpr size_t kZeroedBytes = kWsZeroedBytes;
constexpr size_t kFoldFlagBytes = kWsFoldFlagBytes;
constexpr size_t kFoldFlagOffset = kWsFoldFlagOffset;

struct DeviceInfo {
    std::once_flag once;
    int cus = 256;
};
DeviceInfo g_dev[kMaxDevices];

// Device properties are read once per device; the reference asks the driver
// on every call (marlin_kernel.cu:753).
int compute_units(int dev) {
    if (dev < 0 || dev >= kMaxDevices) return 256;
    DeviceInfo &d = g_dev[dev];
    std::call_once(d.once, [&]() {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
            d.cus = v;
    });
    return d.cus;
}

bool shape_ok(int n, int k, int groupsize) {
    return k % 128 == 0 && n % 256 == 0 && (groupsize == -1 || groupsize == 128);
}

struct DecodePlan {
    int KS, GS, U, BPS, waves;
    bool regs = false;  // for the register-fragment group-major instance
    long cost = -1;
    int gm_tiles = 0;   // > 0: for the LDS-staged group-major instance, tiles per block
    bool gmp = false;   // with gm_tiles > 0: for the private-staging group-major instance
};

enum class DecodeMode { kStaged, kDirect, kRegs };

constexpr int kMaxKSlices = 8;  // bounds the partial-tile workspace
constexpr int kDecodeDirectMaxM = 4;  // rows up to which the decode kernel skips the LDS staging of A

// Overrides of the automatic plan (0 / -1 = automatic).  The shipped library has none: the struct
// is a compile-time constant there and the entry points have no mutable state besides the plan
// cache below.  A second build of this file with -DKILN_W4A16_TUNING_HOOKS (the library the test
// suite and the profiling scripts load for this) makes it a process-wide variable with setters.
struct Tuning {
    int prefill_min_m = 0;            // > 0: the matrix-core kernel takes every GEMM of at least this many rows
    int decode_direct_max_m = -1;
    int decode_group_major = -1;      // 0 = never, 1 = LDS-staged only, 2 = register-fragment wherever it fits
    int decode_runs_per_launch = 0;   // 1 = one run of rows per launch
    int prefill_ks = 0, prefill_bn = 0, prefill_bm = 0, prefill_nb_full = -1;
    int force_ks = 0, force_u = 0, force_waves = 0;
    int gmp_tiles = 0, gmp_waves = 0, gmp_ks = 0;   // > 0: the private-staging small-M instance with this plan
    int mid = -1;                     // 0 = never the mid-M kernel, 1 = wherever a plan fits (any row count), -1 = automatic
    int mid_pairs = 0, mid_ks = 0;    // its tile pairs per block and K slices
    int mid_waves = 0;                // > 0: its wavefronts per block, at most
    int flagged = -1;                 // 0 = K slices always meet through counters, -1 = automatic
    int lora_fold = -1;               // 0 = the LoRA projection always runs as a launch of its own, -1 = automatic,
                                      // 2 = in the launch wherever the kernel can (whatever the grid's size)
    int rowsum_fold = -1;             // 0 = the matrix-core kernel's row sums always come from a launch in front, -1 = automatic
};
#ifdef KILN_W4A16_TUNING_HOOKS
Tuning g_tune;
#else
constexpr Tuning g_tune{};
#endif

// block shape, whole-tile part and slice count the workspace is sized for and the launch starts from
PrefillPlan planned_prefill(int m, int n, int k, int cus) {
    PrefillPlan p = plan_prefill(m, n, k, cus, g_tune.prefill_bn, g_tune.prefill_bm);
    if (g_tune.prefill_nb_full >= 0) p.nb_full = g_tune.prefill_nb_full < n / p.bn ? g_tune.prefill_nb_full : n / p.bn;
    if (g_tune.prefill_ks > 0) {
        const int G = k / kGroupK, ks = g_tune.prefill_ks < G ? g_tune.prefill_ks : G, gsb = (G + ks - 1) / ks;
        p.ks = (G + gsb - 1) / gsb;
    }
    // one arrival counter per sliced tile lives in the counter region
    if ((size_t)((m + p.bm - 1) / p.bm) * (n / p.bn - p.nb_full) * sizeof(int) > kCounterCapacity) p.ks = 1;
    return p;
}

int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Pick the K slicing (KS slices of GS groups), the run length U and the block size.  The model
// behind the cost, fitted to a sweep of the model's projection shapes at M = 1...16 (unit: the
// time one compute unit takes to stream one chunk, about 0.042 us):
//   * every round of blocks costs its chunks per block plus a fixed part (staging the activations,
//     the reduction across wavefronts): about 40 units;
//   * more than one K slice means an exchange of partial tiles through the workspace -- store,
//     arrival counter and read-back are three dependent device-scope round trips, 2.2 us whatever
//     the amount exchanged, plus 0.25 us per slice (partial tiles to write and to add);
//   * blocks that do not hold whole tiles (chunks per block not a multiple of the groups per
//     slice) exchange the cut tiles the same way and double the parts per tile: 2.4-2.7 us.  On the
//     model's shapes whole tiles on fewer compute units beat an even spread over all of them.
//   * Among plans of equal cost, block sizes that give every SIMD the same number of wavefronts
//     (12, 8, 16) go first -- the main loop is bound by vector-instruction issue, so the SIMD
//     with one wavefront more finishes last -- and 12 wavefronts with longer runs measured
//     0.3-0.5 us faster than 15-16 with shorter ones.
// thread_k / thread_n keep the meaning they have in the reference (rows of K / columns of N owned
// by one thread block); -1 picks them here.  `direct`: plan for the kernel instance that reads its
// operand fragments from L2; it stages nothing in LDS, so the slice length has no limit.
//   * Plans that fit the group-major kernel instance (whole tiles, equal slices, groups dividing
//     evenly among the wavefronts) run 0.4-0.8 us faster: fewer products and LDS reads per chunk.
//   * The register-fragment instance reads rows x 256 bytes of activations per group and
//     wavefront from L2.  With one tile per block that is 4 bytes per byte of weights at M = 16
//     (down projection as one slice: 11.1 us against 7.4 us for three slices of two tiles), so
//     its plans need two tiles per block and slices no longer than the staged instances' -- except
//     with few rows and at most two chunks per wavefront, where skipping staging and barrier
//     wins; two slabs of rows double the arithmetic per chunk.
constexpr long kRoundCost = 40, kSliceExchangeCost = 55, kCutTileCost = 60, kGroupMajorGain = 15;
bool plan_decode(int n, int k, int cus, int thread_k, int thread_n, DecodeMode mode, int rows, DecodePlan *out) {
    const bool direct = mode == DecodeMode::kDirect, regs = mode == DecodeMode::kRegs;
    const int G = k / kGroupK, NT = n / kTileN;
    int forced_gs = 0;
    if (thread_k > 0) forced_gs = thread_k / kGroupK < G ? thread_k / kGroupK : G;
    if (g_tune.force_ks) forced_gs = ceil_div(G, g_tune.force_ks);

    static const int kWaveOrder[] = {12, 8, 16, 10, 11, 13, 14, 15, 9, 7, 6, 5, 4};
    long best_cost = -1;
    for (int waves : kWaveOrder) {
        if (g_tune.force_waves ? waves != g_tune.force_waves : waves < 8) continue;
        int gs_cap = (decode_max_lds_bytes() - waves * 2048) / (16 * 256) - 1;
        gs_cap = (direct || regs) ? G : (gs_cap < 32 ? gs_cap : 32);
        for (int ks = 1; ks <= kMaxKSlices && ks <= G; ++ks) {
            int GS = forced_gs ? forced_gs : ceil_div(G, ks);
            if (forced_gs && GS > gs_cap) GS = gs_cap;
            if (forced_gs && ceil_div(G, GS) > kMaxKSlices) GS = ceil_div(G, kMaxKSlices);
            if (GS > gs_cap) continue;
            const int KS = ceil_div(G, GS);
            const int gs_last = G - (KS - 1) * GS;
            if (KS > kMaxKSlices) continue;
            const int u_max = gs_last < decode_max_run() ? gs_last : decode_max_run();
            for (int U = ceil_div(GS, waves); U <= u_max; ++U) {
                if (g_tune.force_u && U != g_tune.force_u) continue;
                if (thread_n > 0 && !g_tune.force_u) {  // columns per block -> chunks per block
                    int want = ceil_div((thread_n / kTileN) * GS, waves);
                    want = want < ceil_div(GS, waves) ? ceil_div(GS, waves) : (want > u_max ? u_max : want);
                    if (U != want) continue;
                }
                const int R = waves * U;
                if (R / gs_last + 2 > decode_max_tiles_per_block()) break;
                const int BPS = ceil_div(NT * GS, R);
                const int rounds = ceil_div(BPS * KS, cus);
                const bool cut = R % GS != 0 || R % gs_last != 0;
                if (regs && (R / GS < 2 || GS > 32) && !(rows <= kDecodeDirectMaxM && U <= 2 && GS <= 32)) continue;
                long cost = (long)rounds * (R * (rows > 16 ? 2 : 1) + kRoundCost) +
                            (KS > 1 ? kSliceExchangeCost + 6 * KS : 0) + (cut ? kCutTileCost : 0);
                const long gm_gain = kGroupMajorGain * (R / GS - 1) / (R / GS > 0 ? R / GS : 1);  // none for one tile
                DecodeArgs probe;
                probe.M = rows;
                probe.K = k;
                probe.KS = KS;
                probe.GS = GS;
                probe.U = U;
                probe.waves = waves;
                probe.direct = direct;
                probe.group_major = g_tune.decode_group_major;
                if (regs) {
                    if (!decode_group_major_regs_ok(probe)) continue;
                    cost -= gm_gain;
                }
                if (best_cost < 0 || cost < best_cost) {
                    best_cost = cost;
                    *out = DecodePlan{KS, GS, U, BPS, waves, regs, cost, 0};
                }
            }
            // LDS-staged group-major plans: T whole tiles per block, the slice's groups dealt to the
            // wavefronts as evenly as they go (12 wavefronts take 20 groups as 8 x 2 + 4 x 1)
            for (int T = 2; T <= 6 && mode == DecodeMode::kStaged && rows <= 16 && thread_n <= 0; ++T) {
                const int U = T * ceil_div(GS, waves);
                if (U > decode_max_run() || (g_tune.force_u && U != g_tune.force_u)) continue;
                DecodeArgs probe;
                probe.M = rows;
                probe.K = k;
                probe.KS = KS;
                probe.GS = GS;
                probe.U = U;
                probe.waves = waves;
                probe.gm_tiles = T;
                probe.group_major = g_tune.decode_group_major;
                if (!decode_group_major_ok(probe)) continue;
                const int BPS = ceil_div(NT, T);
                const int rounds = ceil_div(BPS * KS, cus);
                const long cost = (long)rounds * (T * GS + kRoundCost) + (KS > 1 ? kSliceExchangeCost + 6 * KS : 0) -
                                  kGroupMajorGain * (T - 1) / T;
                if (best_cost < 0 || cost < best_cost) {
                    best_cost = cost;
                    *out = DecodePlan{KS, GS, U, BPS, waves, false, cost, T};
                }
            }
            if (forced_gs) break;
        }
    }
    return best_cost >= 0;
}

// The plan for one slab of m rows, and which kernel instance runs it.  m <= 16: the cheaper of
// the best plan for the LDS-staged instances and the best plan for the register-fragment
// instance (whose slices may be as long as K: no exchange on the down projection), the latter
// handicapped by what the staged group-major instance measured faster on plans both can run.
// 17 <= m <= 32: only the register-fragment instance takes that many rows; false if no plan fits.
constexpr long kRegsHandicap = 8;
// the private-staging group-major instance with a given plan, if the shape takes it
// lora: the plan must also hold for a call with adapters, whatever their ranks (one wavefront more per
// block and the low-rank term's operands in LDS: checked for the largest rank and slice count)
bool gmp_plan(int m, int n, int k, int tiles, int waves, int ks, bool lora, DecodePlan *plan) {
    const int G = k / kGroupK, NT = n / kTileN;
    if (ks < 1 || G % ks != 0 || tiles < 1) return false;
    DecodeArgs a;
    a.M = m;
    a.N = n;
    a.K = k;
    a.KS = ks;
    a.GS = G / ks;
    a.waves = waves < a.GS ? waves : a.GS;
    a.gm_tiles = tiles;
    if (lora) {
        static const uint16_t probe = 0;  // never dereferenced: the check only asks for non-null operands
        a.r_total = 64;
        a.lora_slices = 16;
        a.lora_rows = m;
        a.lora_t = a.lora_b = &probe;
    }
    if (!decode_gmp_ok(a)) return false;
    *plan = DecodePlan{};
    plan->KS = ks;
    plan->GS = a.GS;
    plan->waves = a.waves;
    plan->gm_tiles = tiles;
    plan->U = tiles * ceil_div(a.GS, a.waves);
    plan->BPS = ceil_div(NT, tiles);
    plan->gmp = true;
    return true;
}

// Can ks slices of n columns exchange their 16-row partial tiles in the zeroed region (every slice
// but the last writes there; the polling wavefront reads the parts of the largest slice count, the
// absent ones as zeros, so the region must hold those too)?
bool flagged_exchange_fits(int ks, int n) {
    return g_tune.flagged != 0 && ks > 1 && ks <= kDecodeFlaggedMaxSlices &&
           (size_t)(kDecodeFlaggedMaxSlices - 1) * (n / kTileN) * 256 * sizeof(float) <= kFlaggedBytes - kFoldFlagBytes;
}

// Best plan for the private-staging group-major instance (m <= 16).  Cost in microseconds, fitted
// to sweeps of the model's projection shapes at 1, 4, 8 and 16 rows and checked against sweeps of
// every plan on 24 shapes (those, the side-by-side packs, and 18 of other models: 1536 ... 28672 wide),
// where the plan it picks is 1.4 % slower than the best forced plan on average and 13 % at worst: a launch costs about 2.8 us
// beside its rounds of blocks; a block streams its T * GS KiB of weights at 0.036 us per KiB and
// stages its rows of A from L2 (GS KiB per four rows) at 0.0125 us per KiB -- with 16 rows an
// unsliced down projection stages four times the bytes it streams, which is why it is sliced there
// and not at 4 rows; a wavefront's chunks run one after the other (0.08 us each); the exchange
// between K slices is priced where the cost is formed (down projection at 16 rows in three
// slices: 7.1 us with the parts as their own arrival flags, 8.4 through counters; four, six, eight
// slices through counters 9.2, 9.9, 11.2).  A call with adapters plans for the chip less the blocks
// that project x onto the adapters, so that the projection can ride in the same launch.
bool plan_decode_gmp(int m, int n, int k, int cus, bool lora, DecodePlan *best) {
    const int G = k / kGroupK, NT = n / kTileN;
    // (a caller may name a part of the chip, `sms`: never plan for less than one unit)
    if (lora && g_tune.lora_fold != 0 && cus > lora_project_slices(m, k)) cus -= lora_project_slices(m, k);
    const int a_kib_per_group = m <= 4 ? 1 : (m <= 8 ? 2 : 4);
    // (with adapters a block has one wavefront more, so 14 stand in for the 16 -- 15 main wavefronts and the low-rank
    // term's operands do not fit LDS at 16 rows: 5120 -> 13824 with two adapters in one round of four-tile blocks
    // 10.6 / 12.7 us at 1 / 16 rows against 14.3 / 18.0 in two rounds of two-tile blocks, 5120 -> 27648 20.4 / 23.3 against 26.8 / 29.2)
    const int most = lora ? 14 : 16;
    const int kWaves[] = {12, most, 8};
    float best_cost = -1.f;
    for (int ks = 1; ks <= kMaxKSlices && ks <= G; ++ks) {
        if (G % ks != 0) continue;
        const int GS = G / ks;
        for (int waves : kWaves) {
            for (int T = 1; T <= 6; ++T) {
                // 16 wavefronts only where they take one tile and the same number of groups each
                // (out-projection: 4.9 against 5.3 us with 12), or where 12 cannot form the plan (a
                // wavefront holds at most 16 chunks: 5120 -> 13824 in blocks of four tiles, one round,
                // 8.4 us at one row against 10.4 in two rounds of two-tile blocks); elsewhere they
                // measured 5 to 15 % slower than 12 on the same tiles and slices
                DecodePlan p;
                if (waves == most && (lora || T != 1 || GS % 16 != 0) && gmp_plan(m, n, k, T, 12, ks, lora, &p)) continue;
                if (!gmp_plan(m, n, k, T, waves, ks, lora, &p)) continue;
                const int rounds = ceil_div(ceil_div(NT, T) * ks, cus);
                // The exchange: through counters 0.4 us per slice + 1.2; with the parts as their own
                // arrival flags it grows with the tiles polled, 0.0037 us per (slice - 1) and tile
                // (down projection, 160 tiles: 0.4 / 1.1 / 1.9 us at two / three / four slices;
                // in-projection, 512 tiles: 2.0 us at two; 576 tiles in two slices of five-tile
                // blocks: 7.0 us against 6.1 unsliced), + 0.3 because the unsliced estimates
                // run high.  At up to four rows the additive model puts sliced plans 1 us too low
                // (down projection: 6.7 us in three slices against 5.7 unsliced): + 0.7 there.
                const bool flagged = flagged_exchange_fits(ks, n);
                const float exchange = ks == 1 ? 0.f : (flagged ? 0.4f + 0.0037f * (ks - 1) * NT : 0.4f * ks + 1.2f) +
                                                           (a_kib_per_group == 1 ? 0.7f : 0.f);
                // Every round after the first costs its blocks' start on top (1 us: 4096 -> 14336 at one row
                // 9.8 us in two rounds of two-tile blocks, 7.5 in one round of four-tile blocks).  Eight
                // wavefronts with three or more tiles each measure 3 to 7 % below twelve on the same
                // tiles (fewer partial tiles to add at the end: gate+up at 16 rows 7.9 -> 7.6 us,
                // q|k|v side by side 6.5 -> 6.15); with adapters the twelve stay (not measured).
                float cost = 2.8f + rounds * (0.036f * T * GS + 0.0125f * a_kib_per_group * GS) +
                             0.08f * T * ceil_div(GS, p.waves) + exchange + 1.0f * (rounds - 1);
                if (waves == 8 && T >= 3 && !lora) cost *= 0.95f;
                if (best_cost < 0.f || cost < best_cost - 1e-4f) {
                    best_cost = cost;
                    *best = p;
                }
            }
        }
    }
    return best_cost >= 0.f;
}

// lora: 0 = a call without adapters, 1 = with adapters the private-staging kernel takes (stacked rank a
// multiple of 8), 2 = with other adapters
bool choose_decode(int m, int n, int k, int cus, int thread_k, int thread_n, int lora, DecodePlan *plan,
                   bool *direct) {
    *direct = false;
    if (g_tune.gmp_tiles > 0 && m <= 16 && lora != 2 &&
        gmp_plan(m, n, k, g_tune.gmp_tiles, g_tune.gmp_waves, g_tune.gmp_ks, lora != 0, plan))
        return true;
    // up to 16 rows of a call without overrides (with or without adapters): the private-staging instance
    if (m <= 16 && lora != 2 && thread_k <= 0 && thread_n <= 0 && g_tune.gmp_tiles == 0 && g_tune.decode_group_major == -1 &&
        g_tune.decode_direct_max_m < 0 && !g_tune.force_ks && !g_tune.force_u && !g_tune.force_waves &&
        plan_decode_gmp(m, n, k, cus, lora != 0, plan))
        return true;
    const bool regs_allowed = g_tune.decode_group_major != 0 && g_tune.decode_group_major != 1 && thread_n <= 0;
    if (m > 16) return regs_allowed && plan_decode(n, k, cus, thread_k, thread_n, DecodeMode::kRegs, m, plan);
    if (g_tune.decode_direct_max_m >= 0 && m <= g_tune.decode_direct_max_m) {  // tuning override
        *direct = true;
        return plan_decode(n, k, cus, thread_k, thread_n, DecodeMode::kDirect, m, plan);
    }
    const bool have_staged = plan_decode(n, k, cus, thread_k, thread_n, DecodeMode::kStaged, m, plan);
    DecodePlan rp;
    if (regs_allowed && plan_decode(n, k, cus, thread_k, thread_n, DecodeMode::kRegs, m, &rp) &&
        (!have_staged || g_tune.decode_group_major == 2 || rp.cost + kRegsHandicap < plan->cost ||
         // few rows, one or two chunks per wavefront: no staging and no barrier wins (cfg 0: 3.4 against 3.8 us)
         (m <= kDecodeDirectMaxM && rp.U <= 2 && rp.cost <= plan->cost))) {
        *plan = rp;
        return true;
    }
    if (!have_staged) return false;
    // few rows and short runs: latency-bound launches, where skipping the staging barrier wins
    // (measured: -0.3...-1.0 us at M <= 4 with up to 3 chunks per wavefront, +0.7 us with 6)
    *direct = g_tune.decode_direct_max_m < 0 && m <= kDecodeDirectMaxM && plan->U <= 3 && plan->gm_tiles == 0;
    return true;
}

// The slab plans are pure functions of (rows, n, k, compute units, overrides) and cost 15-25 us
// of host time each, more than the GEMM they plan, so they are kept: a small table behind a
// mutex (the entry points may be entered from several threads at once).
struct SlabKey {
    int m, n, k, cus, thread_k, thread_n, lora;
    bool operator==(const SlabKey &o) const {
        return m == o.m && n == o.n && k == o.k && cus == o.cus && thread_k == o.thread_k && thread_n == o.thread_n &&
               lora == o.lora;
    }
};
struct SlabKeyHash {
    size_t operator()(const SlabKey &key) const {
        size_t h = 1469598103934665603ull;
        for (int v : {key.m, key.n, key.k, key.cus, key.thread_k, key.thread_n, key.lora}) h = (h ^ (size_t)(unsigned)v) * 1099511628211ull;
        return h;
    }
};
struct SlabChoice {
    bool ok = false;
    bool direct = false;
    DecodePlan plan{};
};
std::mutex g_plan_mutex;
std::unordered_map<SlabKey, SlabChoice, SlabKeyHash> g_plan_cache;

SlabChoice slab_choice(int m, int n, int k, int cus, int thread_k, int thread_n, int lora) {
    const SlabKey key{m, n, k, cus, thread_k, thread_n, lora};
    {
        std::lock_guard<std::mutex> lock(g_plan_mutex);
        auto it = g_plan_cache.find(key);
        if (it != g_plan_cache.end()) return it->second;
    }
    SlabChoice c;
    c.ok = choose_decode(m, n, k, cus, thread_k, thread_n, lora, &c.plan, &c.direct);
    std::lock_guard<std::mutex> lock(g_plan_mutex);
    if (g_plan_cache.size() > 4096) g_plan_cache.clear();  // a caller cycling through many shapes
    g_plan_cache.emplace(key, c);
    return c;
}

// Does a GEMM of m rows that the mid-M kernel does not take (plan overrides, adapters of a stacked rank
// that is not a multiple of 8, shapes without a mid-M plan) take the matrix-core kernel?  Below the change-over the rows go through
// the small-M kernels in runs, every launch streaming the weights again.  Where a plan for the
// two-slab small-M instance exists, up to 80 rows go there (runs of 32 rows, up to four per
// launch); measured against the matrix-core kernel's 64-row blocks (16-24 us at any M <= 64) it is
// ahead or level up to 80 rows on all four projection shapes (at 72 rows 28.3 / 27.5 / 18.1 /
// 16.2 us against 32.2 / 27.1 / 18.9 / 18.5) and behind from 96 rows on.  The one exception is the
// widest projection at 49...64 rows, where one round of 64-row blocks (20.1 us) is ahead of two
// runs (20.2...21.0).  Without such a plan the matrix-core kernel starts at 49 rows.
int mid_max_rows(int n, int k, bool lora = false);
bool takes_prefill(int m, int n, int k, int cus) {
    if (g_tune.prefill_min_m > 0) return m >= g_tune.prefill_min_m;
    if (!slab_choice(32, n, k, cus, -1, -1, false).ok) return m >= 49;
    if ((long)n * k > (32L << 20) && m >= 49 && m <= 64) return true;
    // rows beyond the one run the mid-M kernel takes on the largest weights of a long K: three passes of the
    // small-M kernels over 64 MB and more of weights are behind one of the matrix-core kernel
    if (m > mid_max_rows(n, k)) return true;
    return m >= 81;
}

// Everything the dispatcher decides for one call, as a pure function of the shape, the compute
// units and the overrides: kiln_w4a16_workspace_bytes and the launch path both start from it, so
// the workspace is sized for exactly what the call will use.
constexpr int kMaxDecodeLaunches = 16;
struct DecodeLaunch {
    int r0;        // first row
    int M;         // rows per run (<= 32)
    int rows;      // > M: the launch covers this many rows in runs of M (grid z)
    DecodePlan plan;
    bool direct;
};
struct MidPlan {
    bool ok = false;
    int KS = 1, GS = 0, waves = 0, pairs = 1;
    float cost = 0.f;
    bool fold = true;  // with adapters: the projection in the launch's first blocks (where the launch can)
};
struct GemmPlan {
    bool prefill = false;
    PrefillPlan pf{};
    bool mid = false;
    MidPlan mp{};
    int launches = 0;
    DecodeLaunch dl[kMaxDecodeLaunches];
    size_t decode_partial = 0;  // bytes of partial tiles the largest launch exchanges
};

// f32 partial tiles one small-M launch may exchange: per run and K slice two parts of N x 16.
// Plans of whole tiles in one slice exchange nothing.
// Do the K slices of this launch meet in the zeroed region, the parts being their own arrival flags?
bool launch_flagged(const DecodeLaunch &l, int n) { return l.plan.gmp && flagged_exchange_fits(l.plan.KS, n); }

size_t decode_launch_partial_bytes(const DecodeLaunch &l, int n, int k) {
    const DecodePlan &p = l.plan;
    if (launch_flagged(l, n)) return 0;
    bool exchanges = p.KS > 1;
    if (!p.regs && p.gm_tiles == 0) {  // tile-major runs: blocks may cut tiles
        const int G = k / kGroupK, gs_last = G - (p.KS - 1) * p.GS, R = p.waves * p.U;
        exchanges = exchanges || R % p.GS != 0 || R % gs_last != 0;
    }
    if (!exchanges) return 0;
    const int runs = l.rows > l.M ? (l.rows + l.M - 1) / l.M : 1;
    return (size_t)runs * p.KS * 2 * (size_t)n * 16 * sizeof(float);
}

void plan_as_prefill(int m, int n, int k, int cus, int thread_k, int thread_n, GemmPlan *gp) {
    gp->prefill = true;
    gp->launches = 0;
    gp->decode_partial = 0;
    PrefillPlan p = planned_prefill(m, n, k, cus);
    if ((thread_n == 128 || thread_n == 256) && thread_n != p.bn) {  // block columns: whole tiles only
        p.bn = thread_n;
        p.nb_full = n / thread_n;
        p.ks = 1;
    }
    // thread_k asks for a K slice length; it can lower the slice count but never raise it
    if (thread_k > 0) {
        const int G = k / kGroupK, gs = thread_k / kGroupK < G ? thread_k / kGroupK : G;
        const int want = ceil_div(G, gs);
        if (want < p.ks) p.ks = want;
    }
    gp->pf = p;
}

// Rows the mid-M kernel takes on the automatic plan, from sweeps of the three kernels forced on 13 shapes
// (the model's, the side-by-side packs, seven of other models) at 17 ... 320 rows.
// From: 17 rows.  Up to 32 rows it computes one row block of 32 per pass (half the loads of A and half the
// products of its 64-row pass), and with that it leads the two-slab small-M instance from the first row
// beyond 16 on every shape (down projection at 17 / 32 rows 8.4 / 9.1 us against 9.7 / 12.5, out-projection
// 6.4 / 6.7 against 7.8 / 8.4, in-projection 6.6 / 7.2 against 6.7 / 8.4, 4096 -> 14336 12.6 / 13.4 against
// 15.3 / 21.2) but the wide outputs of a short K (K <= 3072, N >= 10240), which stay with the two-slab instance up
// to 20 rows: the mid-M kernel's time hardly grows with the rows of a run of up to 32 (gate+up 9.8 / 10.1 /
// 10.4 us at 17 / 24 / 32 rows; all three pairs of a block meet in one phase there), the two-slab instance's
// does (9.6 / 10.5 / 11.2), and they cross at 20...21 rows on gate+up, 2560 -> 10240 and 12288 and 2048 -> 11008
// (3584 -> 18944 was level, 19.2...19.6 us, until its 28 groups could go to ten wavefronts unsliced: 12.1 /
// 13.1 us at 17 / 32 rows against 20.8 on the two-slab instance, hence the bound on K).  With adapters 17
// everywhere: the two-slab instance needs the projection from a launch in front, the mid-M kernel computes it
// in its own first blocks (two adapters at 24 rows, out- / in- / down- / gate+up projection: 10.4 / 10.7 /
// 13.4 / 13.7 us against 14.4 / 13.3 / 19.2 / 17.0).
// To: 128 rows (two runs of 64); small weights keep it ahead of the matrix-core kernel's 64-row blocks for
// longer -- K * N up to 32 M: 192 rows, 256 where K <= 4096 (in-projection at 256 rows 25.2 against 26.5 us,
// 2560 -> 12288 31.8 against 35.0, down projection at 192 rows 24.5 against 29.1 but 34.5 against 31.3 at 256);
// up to 12 M: 320 rows (out-projection at 320 rows 16.1 against 23.1, 2560 -> 1024 8.7 against 16.2), up to 9 M:
// 512, up to 2.5 M: 1024 (mid_max_rows) -- while
// on large ones it falls behind from 160 rows on (14336 -> 4096: 55 against 47 us; gate+up 42.5 against 35.2).
constexpr int kMidMinM = 17, kMidMinMWideShortK = 21, kMidMaxM = 128, kMidMaxMSmallest = 320, kMidMaxMTiny = 512, kMidMaxMVerySmallest = 1024;
int mid_min_rows(int n, int k, bool lora) { return !lora && k <= 3072 && n >= 10240 ? kMidMinMWideShortK : kMidMinM; }
static int mid_max_rows_by_weights(int n, int k, bool lora);
int mid_max_rows(int n, int k, bool lora) {
    int rows = mid_max_rows_by_weights(n, k, lora);
    // Wide outputs of a short K: the kernel's time there is its blocks' starts, meetings and stores, one set per
    // 64 rows and pair of tiles, and the matrix-core kernel's wider blocks overtake it at about 2.1 M (K < 1536) or
    // 3.2 M output elements whatever the weights' size (896 -> 9728, 8.7 M weights: 13.3 us at 192 rows against 16.3,
    // but 19.5 / 28.0 / 36.4 at 256 / 384 / 512 against 16.2 / 17.2 / 22.1; 1536 -> 17920 at 192 rows 31.7 against
    // 23.1; 3584 -> 37888 at 96 / 128 rows 58 / 70 against 56 / 57, with adapters 81 / 97 against 58; while
    // 2560 -> 12288 and 2048 -> 11264 at 256 rows lead by 9 %: 31.8 against 35.0, 26.9 against 29.6)
    // (K = 4096 included: 4096 -> 28672 at 128 rows 68 us against 58 on the matrix-core kernel, with two adapters 78
    // against 56, while 4096 -> 22016, 2.8 M output elements there, leads with 49 against 67)
    if (k <= 4096) {
        const int cap = (int)((k < 1536 ? 2100000ll : 3200000ll) / n / 64 * 64);
        rows = std::min(rows, std::max(cap, mid_max_rows_per_run()));
    }
    return rows;
}
static int mid_max_rows_by_weights(int n, int k, bool lora) {
    const long long kn = (long long)k * n;
    // the very smallest: to 1024 rows (1024 -> 1024 at 640...1024 rows 6.4...6.6 us against 13.4...14.6 on the
    // matrix-core kernel, 1536 -> 1536 8.7...11.3 against 17...18.5, 2560 -> 1024 11.8...14.6 against 18.5...20; at 4 M
    // 2048 -> 2048 and 4096 -> 1024 still lead by a sixth there but 1024 -> 4096 is behind from 640 on).
    // Calls with adapters keep the 320 rows they were measured at.
    if (kn <= 5ll << 19 && !lora) return kMidMaxMVerySmallest;
    // the smallest weights: to 512 rows (at 448...512 rows 2560 -> 1024 9.2...9.4 us against 17.1...17.5 on the
    // matrix-core kernel, 2048 -> 2048 9.8 against 18, 4096 -> 1024 12.3...12.7 against 22...23, 3072 -> 3072 17.2...17.8
    // against 26; 4096 -> 2560, 10 M, is behind there: 29.7 against 26.2)
    if (kn <= 9ll << 20 && !lora) return kMidMaxMTiny;
    if (kn <= 12ll << 20) return kMidMaxMSmallest;
    if (kn <= 32ll << 20) return k <= 4096 ? 256 : 192;
    // the largest weights with a long K: one run of rows (at 96 / 128 rows 8192 -> 8192 37.2 / 39.3 us against
    // 37.2 / 36.3 on the matrix-core kernel, 5120 -> 13824 46.9 / 48.1 against 40.8 / 40.4, 13824 -> 5120 42.8 /
    // 45.0 against 39.9 / 39.2, 18944 -> 3584 46.9 against 41.2 at 128; 3584 -> 18944, as large but of a short K,
    // 39 / 40 against 50, and 14336 -> 4096, 56 M, level)
    if (kn > 60ll << 20 && k >= 5120) return mid_max_rows_per_run();
    return kMidMaxM;
}

// Do the K slices of this mid-M launch meet in the zeroed region, the parts being their own arrival flags?
bool mid_flagged(const MidArgs &a) {
    // the last slice polls kMidFlaggedSlices - 1 parts whatever KS is: up to one slice's parts past the launch's own
    return g_tune.flagged != 0 && mid_flagged_ok(a) &&
           mid_partial_bytes(a) / a.KS * (a.KS + 1) <= kFlaggedBytes - kFoldFlagBytes;
}

// Plan for the mid-M kernel: pairs of tiles per block, K slices, wavefronts.  Cost in microseconds,
// fitted to a sweep of the four projection shapes at 33...192 rows (and checked from 17 on, see below): a wavefront's group step is
// bound by the round trip of its activations through L2 and by the products of its pairs
// (0.75 + 0.55 us per pair; every block re-reads its rows of A, so fewer and wider blocks trade
// parallelism for L2 traffic); a launch costs about 4.5 us beside its rounds of blocks, an exchange
// between K slices through counters 1.5 us at two slices and 1.7 us more per further slice
// (out-projection at 64 rows: 11.5 us unsliced, 10.4 in two slices, 13.8 in four), the counter-free
// exchange 1 us less at two slices (9.4) and 0.5 us per further slice (the four-slice figure above held a
// second round of blocks; 4096 -> 1024, 128 blocks in four slices: 6.4 us at 64 rows against 7.9 in two).
// Every round of blocks after the first costs its start on top (2 us: without it many rounds of short
// slices looked cheap -- 5120 -> 13824 at 128 rows 58 us in five slices against 48 in two).  Checked
// against every forced plan on 22 shapes (those four, the side-by-side packs and 16 of other models) at
// 17, 32, 40, 64, 96 and 128 rows: the plan picked is 0.4 % slower than the best on average from 40 rows
// on and 1.3 % at 17 and 32, 10 % at worst where the automatic route takes this kernel (3584 -> 18944 at
// 40 rows, 4096 -> 11008 at 17: three pairs in two slices where two pairs unsliced would lead).  Eight
// narrow outputs of a long K swept afterwards (4096 -> 512 ... 8192 -> 3072 at 24, 64 and 128 rows): within
// 4 % of the best plan but on 6144 -> 1536 (6...12 %: 12 groups dealt to 8 wavefronts count as 16).
MidPlan plan_mid_waves(int m, int n, int k, int cus, bool lora, bool ten_beyond_32_rows) {
    MidPlan best;
    const int G = k / kGroupK, runs = ceil_div(m, mid_max_rows_per_run());
    for (int pairs = 1; pairs <= 3; ++pairs) {
        if (g_tune.mid_pairs && pairs != g_tune.mid_pairs) continue;
        for (int ks = 1; ks <= kMaxKSlices && ks <= G; ++ks) {
            // (a shorter last slice: not in the plan of last resort below, which was not measured with one)
            if ((G % ks != 0 && ten_beyond_32_rows) || (g_tune.mid_ks && ks != g_tune.mid_ks)) continue;
            MidArgs a{};
            a.M = m;
            a.N = n;
            a.K = k;
            a.KS = ks;
            a.GS = ceil_div(G, ks);  // the last slice may be shorter (mid_plan_ok says when)
            // Ten wavefronts where a launch may have them (up to 32 rows, or one pair per block without adapters) and eight
            // would take four groups each or more: 5120 -> 13824 at 17...32 rows 16.7...17.3 us (eight cannot
            // hold 40 groups: two slices) -> 13.0...13.9, 4096 -> 14336 12.0...12.4 -> 11.6...12.0.  Not below:
            // 20 groups as 10 x 2 measured 2...9 % slower than as 4 x 3 + 4 x 2 (in-projection 6.4 -> 6.5 us,
            // 2560 -> 2560 5.5 -> 5.85), the shorter main loop paid for by the start and the meeting of more wavefronts.
            // Beyond 32 rows only blocks of one pair may have ten, and the 64-row pass with four groups to a
            // wavefront waits for A more than this model knows (13824 -> 5120 at 64 rows 29.9 us in three slices
            // of 10 x 4 against 26.0 in six of 8 x 3; 5120 -> 5120 15.2 against 13.1): there they are the plan of
            // last resort (plan_mid).
            int max_waves = a.GS > 24 && (m <= 32 || ten_beyond_32_rows) ? mid_max_waves(m, pairs, lora) : 8;
            // (with adapters in plans of one or two slices only: 5120 -> 13824 with two adapters at 17 rows 19.3 -> 15.1 us
            // unsliced, 9216 -> 2560 13.1 -> 12.0 and 8192 -> 8192 21.0 -> 19.8 in two slices, but 13824 -> 5120 in three
            // slices of 6 x 4 + 4 x 3 groups 22.2 against 20.0 in four slices of eight wavefronts)
            if (lora && ks > 2) max_waves = 8;
            if (g_tune.mid_waves > 0) max_waves = std::min(g_tune.mid_waves, mid_max_waves(m, pairs, lora));
            a.waves = a.GS < max_waves ? a.GS : max_waves;
            a.pairs = pairs;
            if (!mid_plan_ok(a)) continue;
            const int col_blocks = mid_column_blocks(a);
            if ((size_t)runs * col_blocks * sizeof(int) > kCounterCapacity) continue;
            const int gpw = ceil_div(a.GS, a.waves), rounds = ceil_div(col_blocks * ks * runs, cus);
            const float exchange = ks == 1 ? 0.f : (mid_flagged(a) ? 0.5f * ks - 0.5f : 1.7f * ks - 1.9f);
            // (a shorter last slice where even ones are clearly worse or do not exist: 13824 -> 5120 at 64 rows runs
            // 26.6 us in six even slices and 28.4...30.1 in five of 22 + 22 + 22 + 22 + 20 groups, which this model
            // would prefer by the 1.7 us of a slice's exchange)
            const float uneven = G % ks != 0 ? 2.0f : 0.f;
            const float cost = rounds * gpw * (0.75f + 0.55f * pairs) + 4.5f + exchange + 2.0f * (rounds - 1) + uneven;
            if (!best.ok || cost < best.cost) {
                best.ok = true;
                best.KS = ks;
                best.GS = a.GS;
                best.waves = a.waves;
                best.pairs = pairs;
                best.cost = cost;
            }
        }
    }
    return best;
}

// The plan of eight wavefronts (ten up to 32 rows); where none exists -- 18944 = 148 groups = 4 x 37 -- and the
// launch is one run of rows, one with ten wavefronts on blocks of one pair: 18944 -> 3584 at 48 / 64 rows 31 us
// against 40.5 on the matrix-core kernel (at 128 rows 60 against 43: not beyond one run).
MidPlan plan_mid(int m, int n, int k, int cus, bool lora) {
    const MidPlan plan = plan_mid_waves(m, n, k, cus, lora, false);
    if (plan.ok || m <= 32 || m > mid_max_rows_per_run()) return plan;
    return plan_mid_waves(m, n, k, cus, lora, true);
}

MidArgs mid_args(const MidPlan &mp, int m, int n, int k) {
    MidArgs a{};
    a.M = m;
    a.N = n;
    a.K = k;
    a.KS = mp.KS;
    a.GS = mp.GS;
    a.waves = mp.waves;
    a.pairs = mp.pairs;
    a.flagged = mid_flagged(a);
    return a;
}

void plan_gemm(int m, int n, int k, int cus, int thread_k, int thread_n, int lora, GemmPlan *gp) {
    *gp = GemmPlan{};
    // mid_min_rows() ... mid_max_rows() rows: the mid-M kernel, one pass over the weights per 64 rows (with
    // adapters whose stacked rank is a multiple of 8: the low-rank term is added from a projection that runs
    // in the launch's first blocks where it fits, else from one launched in front)
    // (a call pinned to a block shape of the matrix-core kernel goes there)
    const bool prefill_pinned = g_tune.prefill_bm != 0 || g_tune.prefill_bn != 0 || g_tune.prefill_ks != 0 || g_tune.prefill_nb_full >= 0;
    // (with adapters also below 17 rows where the small-M launch would have to take the projection from a launch in
    // front -- its blocks fill the chip and leave the producers no units of their own -- and this kernel need not:
    // 11008 -> 4096, 256 blocks of two tiles in two slices, with two adapters 15.3...17.0 us at 1...16 rows, here 13.9...14.4)
    bool few_rows_here = false;
    if (lora == 1 && m <= 16 && g_tune.lora_fold != 0 && g_tune.lora_fold != 2 && g_tune.gmp_tiles == 0 && thread_k <= 0 && thread_n <= 0) {
        DecodePlan dp;
        if (plan_decode_gmp(m, n, k, cus, true, &dp)) {
            const int steps = k / 32, kz0 = lora_project_slices(m, k), per = ((steps + kz0 - 1) / kz0 + 3) / 4 * 4;
            const int kz = (steps + per - 1) / per, blocks = dp.BPS * dp.KS;
            few_rows_here = blocks <= cus && blocks + kz > cus;
        }
    }
    if (lora != 2 && thread_k <= 0 && thread_n <= 0 && g_tune.mid != 0 &&
        (g_tune.mid == 1 ||
         (!prefill_pinned && g_tune.prefill_min_m == 0 && (m >= mid_min_rows(n, k, lora != 0) || few_rows_here) &&
          m <= mid_max_rows(n, k, lora != 0)))) {
        // with adapters the projection runs in the launch's first blocks: plan for the chip less those
        const int producers = lora && g_tune.lora_fold != 0 ? ceil_div(m, 16) * lora_project_slices(m, k) : 0;
        MidPlan mp = plan_mid(m, n, k, cus > 2 * producers ? cus - producers : cus, lora != 0);
        // ... unless the plan for the whole chip is ahead by more than the projection's own launch costs (3 us: what
        // calls of one plan either way differ by) -- where the product's blocks just fill the chip, the producers push
        // the plan into another round or another shape: 2560 -> 12288 with two adapters at 128 rows, 128 blocks
        // of three pairs per run, 26.6 us folded against 22.7 in front; 3584 -> 37888 at 96 rows 81 against 68
        if (producers > 0 && cus > 2 * producers && g_tune.lora_fold != 2) {
            MidPlan whole = plan_mid(m, n, k, cus, true);
            if (whole.ok && (!mp.ok || whole.cost + 3.0f < mp.cost)) {
                whole.fold = false;
                mp = whole;
            }
        }
        if (mp.ok) {
            gp->mid = true;
            gp->mp = mp;
            return;
        }
    }
    // the small-M kernels keep one arrival counter per column tile (and run) in the counter region
    const bool counters_fit = (size_t)(n / kTileN) * sizeof(int) <= kCounterCapacity;
    if (!counters_fit || takes_prefill(m, n, k, cus)) return plan_as_prefill(m, n, k, cus, thread_k, thread_n, gp);
    // Runs of A, one launch each -- launches on one stream run in order, so they may share the
    // workspace -- of 16 rows, or of up to 32 where the plan fits the kernel instance that takes two
    // 16-row slabs in one pass over the weights; where more than 32 rows are left and that
    // instance runs, up to four runs of 32 share one launch (a later run's blocks fill the units the
    // earlier ones leave idle; each run has its own counters and partial tiles).
    // the private-staging kernel takes adapters only where one launch covers the whole call (it reads T whole)
    const int slab_lora = (lora == 1 && m > 16) ? 2 : lora;
    for (int r0 = 0; r0 < m;) {
        if (gp->launches == kMaxDecodeLaunches) return plan_as_prefill(m, n, k, cus, thread_k, thread_n, gp);
        DecodeLaunch &l = gp->dl[gp->launches];
        const int left = m - r0;
        l.r0 = r0;
        l.M = left < 32 ? left : 32;
        SlabChoice c;
        if (l.M > 16) c = slab_choice(l.M, n, k, cus, thread_k, thread_n, slab_lora);
        if (!c.ok) {
            l.M = left < 16 ? left : 16;
            c = slab_choice(l.M, n, k, cus, thread_k, thread_n, slab_lora);
            // no small-M plan (K beyond eight slices of 32 groups): the matrix-core kernel takes any M
            if (!c.ok) return plan_as_prefill(m, n, k, cus, thread_k, thread_n, gp);
        }
        l.plan = c.plan;
        l.direct = c.direct;
        l.rows = 0;
        int max_runs = kMaxKSlices / l.plan.KS < 4 ? kMaxKSlices / l.plan.KS : 4;
        if ((size_t)max_runs * (n / kTileN) * sizeof(int) > kCounterCapacity) max_runs = 1;
        if (g_tune.decode_runs_per_launch > 0 && max_runs > g_tune.decode_runs_per_launch)
            max_runs = g_tune.decode_runs_per_launch;
        int step = l.M;
        if (l.M == 32 && l.plan.regs && left > 32 && max_runs >= 2) {
            l.rows = left < 32 * max_runs ? left : 32 * max_runs;
            step = l.rows;
        }
        const size_t pb = decode_launch_partial_bytes(l, n, k);
        if (pb > gp->decode_partial) gp->decode_partial = pb;
        ++gp->launches;
        r0 += step;
    }
}

// workspace of one call: counters | small-M partial tiles | LoRA projection             (small-M path)
//                        counters | row-sum operands | partial tiles | LoRA projection (matrix-core path)
// The LoRA projection's scratch comes last: a call without adapters needs `plain` bytes only.
struct WorkspaceLayout {
    size_t decode_partial, aext, lora_t, prefill_partial, plain, total;
};
WorkspaceLayout workspace_layout(const GemmPlan &gp, int m, int n, int k) {
    WorkspaceLayout w{};
    size_t off = kZeroedBytes;
    if (gp.prefill) {
        w.aext = off;
        off += prefill_aext_bytes(m, k);
        off = (off + 255) & ~(size_t)255;
        w.prefill_partial = off;
        off += prefill_partial_bytes(m, n, gp.pf);
    } else {
        w.decode_partial = off;
        if (gp.mid) {
            const MidArgs ma = mid_args(gp.mp, m, n, k);
            if (ma.flagged) w.decode_partial = kCounterBytes;  // in the zeroed region, nothing behind it
            else off += mid_partial_bytes(ma);
        } else {
            off += gp.decode_partial;
        }
    }
    w.plain = off;
    off = (off + 255) & ~(size_t)255;
    w.lora_t = off;
    off += prefill_lora_t_bytes(m, !gp.prefill);
    w.total = off;
    return w;
}

__global__ void dequant_f32_kernel(const u32x4 *__restrict__ B, const uint16_t *__restrict__ S,
                                   float *__restrict__ out, int K, int N, int Gs) {
    const int G = K / kGroupK;
    const int chunk = blockIdx.x;  // nt * G + g
    const int nt = chunk / G, g = chunk % G;
    const int lane = threadIdx.x;
    const int c = lane & 15, kq = lane >> 4;
    const u32x4 w = B[(size_t)chunk * 64 + lane];
    const float s = f16_bits_to_f32(S[scale_index(Gs == 1 ? 0 : g, nt * kTileN + c, Gs)]);
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int code = (words[t] >> (4 * nibble_pos(j))) & 0xF;
            const int kk = g * kGroupK + 32 * t + 8 * kq + j;
            out[(size_t)kk * N + nt * kTileN + c] = (float)(code - 8) * s;   // lib.rs:425
        }
}

// zero-fill in 16-byte units (a kernel, not a memset: callers may record it into a graph)
__global__ void zero_fill_kernel(u32x4 *__restrict__ dst, size_t units) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < units; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = u32x4{0u, 0u, 0u, 0u};
}

}  // namespace

}  // namespace kiln

using namespace kiln;

namespace kiln {
namespace {

struct LoraSpec {
    const void *a;       // bf16 [r_total, K]
    const void *b;       // bf16 [N, r_total]
    int r_total, n_adapters;
    const int *ranks;    // host arrays of length n_adapters
    const float *scales;
};

// Bytes a call of m rows needs, made monotone in m: the largest need of any m' <= m.  The plan
// (and with it the need) changes with m' only through the small-M and mid-M runs (m' <= 1024 here; beyond
// that only overrides keep a call on that path) and through the matrix-core kernel's row blocks
// of 64 or 128 rows, so those m' are the ones evaluated.
#ifndef KILN_W4A16_TUNING_HOOKS
// What workspace_bytes_upto found, by its arguments: the sizing walks over hundreds of plans (0.35...0.55 ms
// of host time from 512 rows on), and callers that size per call -- the Python wrappers do -- ask for the
// same few shapes again and again.  Not in the tuning build, whose overrides change the answer.
struct SizeKey {
    int m, n, k, cus, thread_k, thread_n;
    bool operator==(const SizeKey &o) const {
        return m == o.m && n == o.n && k == o.k && cus == o.cus && thread_k == o.thread_k && thread_n == o.thread_n;
    }
};
struct SizeKeyHash {
    size_t operator()(const SizeKey &s) const {
        size_t h = 1469598103934665603ull;
        for (int v : {s.m, s.n, s.k, s.cus, s.thread_k, s.thread_n}) h = (h ^ (size_t)(unsigned)v) * 1099511628211ull;
        return h;
    }
};
std::mutex g_size_mutex;
std::unordered_map<SizeKey, size_t, SizeKeyHash> g_size_cache;
#endif

size_t workspace_bytes_upto(int m, int n, int k, int cus, int thread_k, int thread_n) {
#ifndef KILN_W4A16_TUNING_HOOKS
    const SizeKey key{m, n, k, cus, thread_k, thread_n};
    {
        std::lock_guard<std::mutex> lock(g_size_mutex);
        auto it = g_size_cache.find(key);
        if (it != g_size_cache.end()) return it->second;
    }
#endif
    size_t most = 0;
    auto consider = [&](int mm) {
        for (int lora = 0; lora < 3; ++lora) {  // a call with adapters may take another path
            GemmPlan gp;
            plan_gemm(mm, n, k, cus, thread_k, thread_n, lora, &gp);
            const size_t need = workspace_layout(gp, mm, n, k).total;
            if (need > most) most = need;
        }
    };
    const int small = g_tune.prefill_min_m > kMidMaxMVerySmallest ? g_tune.prefill_min_m : kMidMaxMVerySmallest;
    for (int mm = 1; mm <= m && mm <= small; ++mm) consider(mm);
    for (int mm = 64; mm < m; mm += 64) consider(mm);
    consider(m);
#ifndef KILN_W4A16_TUNING_HOOKS
    std::lock_guard<std::mutex> lock(g_size_mutex);
    if (g_size_cache.size() > 4096) g_size_cache.clear();  // a caller cycling through many shapes
    g_size_cache.emplace(key, most);
#endif
    return most;
}

// The GEMM behind every entry point: small-M or matrix-core path by row count, with the
// optional low-rank term.
kiln_marlin_status_t gemm_any(const void *A, const void *B, void *C, const void *s, int prob_m, int prob_n,
                              int prob_k, void *workspace, int groupsize, int dev, void *stream, int thread_k,
                              int thread_n, int sms, const LoraSpec *lora, bool swiglu = false) {
    if (prob_m < 0 || prob_n < 0 || prob_k < 0) return KILN_W4A16_ERR_PROB_SHAPE;
    if (!shape_ok(prob_n, prob_k, groupsize)) return KILN_W4A16_ERR_PROB_SHAPE;
    if (thread_k > 0 && thread_k % 128 != 0) return KILN_W4A16_ERR_PROB_SHAPE;
    if (thread_n > 0 && thread_n % 16 != 0) return KILN_W4A16_ERR_PROB_SHAPE;
    if (prob_m == 0 || prob_n == 0 || prob_k == 0) return KILN_W4A16_OK;  // marlin_kernel.cu:772-773
    if (!A || !B || !C || !s || !workspace) return KILN_W4A16_ERR_ARGUMENT;
    // the kernels move every operand in 16-byte pieces (rows of A and C are multiples of 256 and 512 bytes)
    for (const void *p : {A, B, static_cast<const void *>(C), s, static_cast<const void *>(workspace)})
        if (reinterpret_cast<uintptr_t>(p) % 16 != 0) return KILN_W4A16_ERR_ARGUMENT;

    const int cus = sms > 0 ? sms : compute_units(dev);
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    GemmPlan gp;
    const int lora_kind = !lora ? 0 : (lora->r_total % 8 == 0 ? 1 : 2);
    plan_gemm(prob_m, prob_n, prob_k, cus, thread_k, thread_n, lora_kind, &gp);
    const WorkspaceLayout wl = workspace_layout(gp, prob_m, prob_n, prob_k);
    char *ws = reinterpret_cast<char *>(workspace);
    char *lora_t = ws + wl.lora_t;
    if (gp.prefill) {
        PrefillArgs pa{};
        pa.A = A;
        pa.B = B;
        pa.S = s;
        pa.C = C;
        pa.aext = ws + wl.aext;
        pa.M = prob_m;
        pa.N = prob_n;
        pa.K = prob_k;
        pa.Gs = (groupsize == -1) ? 1 : prob_k / kGroupK;
        if (lora) {
            pa.lora_t = lora_t;
            pa.lora_a = lora->a;
            pa.lora_b = lora->b;
            pa.r_total = lora->r_total;
            pa.n_adapters = lora->n_adapters;
            pa.ranks = lora->ranks;
            pa.scales = lora->scales;
            if (g_tune.lora_fold != 0) pa.lora_words = reinterpret_cast<unsigned *>(ws + kFoldFlagOffset);
        } else if (g_tune.rowsum_fold != 0) {
            pa.lora_words = reinterpret_cast<unsigned *>(ws + kFoldFlagOffset);
        }
        pa.swiglu = swiglu;
        pa.cus = cus;
        pa.KS = gp.pf.ks;
        pa.bn = gp.pf.bn;
        pa.bm = gp.pf.bm;
        pa.nb_full = gp.pf.nb_full;
        pa.counters = reinterpret_cast<int *>(workspace);
        pa.partial = reinterpret_cast<float *>(ws + wl.prefill_partial);
        return launch_prefill(pa, st) == hipSuccess ? KILN_W4A16_OK : KILN_W4A16_ERR_LAUNCH;
    }

    if (gp.mid) {
        MidArgs ma = mid_args(gp.mp, prob_m, prob_n, prob_k);
        ma.A = A;
        ma.B = B;
        ma.S = s;
        ma.C = C;
        ma.Gs = (groupsize == -1) ? 1 : prob_k / kGroupK;
        ma.swiglu = swiglu;
        ma.counters = reinterpret_cast<int *>(workspace);
        ma.partial = reinterpret_cast<float *>(ws + wl.decode_partial);
        if (lora) {  // the scaled projection of all rows onto the adapters, in K slices
            ma.lora_t = lora_t;
            ma.lora_b = lora->b;
            ma.r_total = lora->r_total;
            // ... inside the product's launch where its blocks have the threads for it: the projection's blocks
            // are the grid's first, so they run before anything that waits for them, in one round or several
            // (gate+up with two adapters at 96 rows 34.9 -> 32.0 us, down 23.7 -> 20.5)
            const int steps = prob_k / 32, row_tiles = ceil_div(prob_m, 16);
            int kz = lora_project_slices(prob_m, prob_k);
            const int per_slice = ((steps + kz - 1) / kz + 3) / 4 * 4;  // whole 128-value groups
            kz = (steps + per_slice - 1) / per_slice;
            MidArgs folded = ma;
            folded.lora_slices = kz;
            folded.lora_producers = row_tiles * kz;
            folded.lora_steps_per_slice = per_slice;
            folded.lora_a = lora->a;
            folded.lora_words = reinterpret_cast<unsigned *>(ws + kFoldFlagOffset);
            folded.lora_adapters = lora->n_adapters;
            // (what the launch itself checks: beyond four runs of rows, or more (slice, tile) words than a copy
            // holds, the projection runs in front -- a call of 320 rows with adapters was refused here once)
            if (g_tune.lora_fold != 0 && gp.mp.fold && lora->n_adapters <= 8 && mid_lora_fold_ok(folded)) {
                int end = 0;
                for (int i = 0; i < 8; ++i) {
                    if (i < lora->n_adapters) end += lora->ranks[i];
                    folded.lora_ends[i] = end;
                    folded.lora_scales[i] = i < lora->n_adapters ? lora->scales[i] : 0.f;
                }
                return launch_mid(folded, st) == hipSuccess ? KILN_W4A16_OK : KILN_W4A16_ERR_LAUNCH;
            }
            PrefillArgs pj{};
            pj.A = A;
            pj.M = prob_m;
            pj.K = prob_k;
            pj.lora_t = lora_t;
            pj.lora_a = lora->a;
            pj.r_total = lora->r_total;
            pj.n_adapters = lora->n_adapters;
            pj.ranks = lora->ranks;
            pj.scales = lora->scales;
            int slices = 1;
            if (launch_lora_project(pj, true, st, &slices) != hipSuccess) return KILN_W4A16_ERR_LAUNCH;
            ma.lora_slices = slices;
        }
        return launch_mid(ma, st) == hipSuccess ? KILN_W4A16_OK : KILN_W4A16_ERR_LAUNCH;
    }

    int rp = 0, lora_slices = 1;
    // Up to 16 rows on the private-staging kernel: the projection rides in the GEMM launch (extra
    // blocks at the front of its grid) instead of running as a launch of its own.
    DecodeArgs fold_probe{};
    bool fold = false;
    int fold_steps = 0;
    if (lora && g_tune.lora_fold != 0 && gp.launches == 1 && gp.dl[0].plan.gmp && gp.dl[0].M == prob_m) {
        const int steps = prob_k / 32;
        int kz = lora_project_slices(prob_m, prob_k);
        fold_steps = ((steps + kz - 1) / kz + 3) / 4 * 4;  // whole 128-value groups, as the projection launch cuts them
        kz = (steps + fold_steps - 1) / fold_steps;
        fold_probe.M = prob_m;
        fold_probe.K = prob_k;
        fold_probe.KS = gp.dl[0].plan.KS;
        fold_probe.GS = gp.dl[0].plan.GS;
        fold_probe.waves = gp.dl[0].plan.waves;
        fold_probe.gm_tiles = gp.dl[0].plan.gm_tiles;
        fold_probe.r_total = lora->r_total;
        fold_probe.lora_a = lora->a;
        fold_probe.lora_t = lora_t;
        fold_probe.lora_flags = reinterpret_cast<unsigned *>(ws + kFoldFlagOffset);
        fold_probe.lora_producers = fold_probe.lora_slices = kz;
        fold_probe.lora_steps_per_slice = fold_steps;
        fold_probe.lora_rows = prob_m;
        fold_probe.lora_adapters = lora->n_adapters;
        // the producers take compute units of their own: where the launch still fits the chip in one round
        // (the in-projection's 256 blocks do not: 12.6 us folded against 10.6 with the launch of its own), or
        // runs in several rounds anyway (5120 -> 13824, 432 blocks: 14.8 us folded against 18.8)
        const int blocks = gp.dl[0].plan.BPS * gp.dl[0].plan.KS;
        fold = decode_gmp_fold_ok(fold_probe) && (blocks + kz <= cus || blocks > cus || g_tune.lora_fold == 2);
        if (fold) {
            lora_slices = kz;
            rp = (lora->r_total + 15) / 16 * 16;
        }
    }
    if (lora && !fold) {  // the scaled projection of all rows onto the adapters, once, ahead of the runs
        PrefillArgs pj{};
        pj.A = A;
        pj.M = prob_m;
        pj.K = prob_k;
        pj.lora_t = lora_t;
        pj.lora_a = lora->a;
        pj.r_total = lora->r_total;
        pj.n_adapters = lora->n_adapters;
        pj.ranks = lora->ranks;
        pj.scales = lora->scales;
        if (launch_lora_project(pj, true, st, &lora_slices) != hipSuccess) return KILN_W4A16_ERR_LAUNCH;
        rp = (lora->r_total + 15) / 16 * 16;
    }
    DecodeArgs a;
    a.B = B;
    a.S = s;
    a.counters = reinterpret_cast<int *>(workspace);
    a.partial = reinterpret_cast<float *>(ws + wl.decode_partial);
    a.N = prob_n;
    a.K = prob_k;
    a.Gs = (groupsize == -1) ? 1 : prob_k / kGroupK;
    a.swiglu = swiglu;
    const int ldc = swiglu ? prob_n / 2 : prob_n;  // the fused gate/up result is half as wide
    for (int i = 0; i < gp.launches; ++i) {
        const DecodeLaunch &l = gp.dl[i];
        a.A = reinterpret_cast<const uint16_t *>(A) + (size_t)l.r0 * prob_k;
        a.C = reinterpret_cast<uint16_t *>(C) + (size_t)l.r0 * ldc;
        if (lora) {
            a.lora_t = reinterpret_cast<const uint16_t *>(lora_t) + (size_t)l.r0 * rp;
            a.lora_b = lora->b;
            a.r_total = lora->r_total;
            a.lora_slices = lora_slices;
            a.lora_rows = prob_m;
            if (fold) {
                a.lora_producers = lora_slices;
                a.lora_steps_per_slice = fold_steps;
                a.lora_a = lora->a;
                a.lora_flags = fold_probe.lora_flags;
                a.lora_adapters = lora->n_adapters;
                int end = 0;
                for (int j = 0; j < 4; ++j) {
                    if (j < lora->n_adapters) end += lora->ranks[j];
                    a.lora_ends[j] = end;
                    a.lora_scales[j] = j < lora->n_adapters ? lora->scales[j] : 0.f;
                }
            }
        }
        a.M = l.M;
        a.rows = l.rows;
        a.direct = l.direct;
        a.KS = l.plan.KS;
        a.GS = l.plan.GS;
        a.U = l.plan.U;
        a.BPS = l.plan.BPS;
        a.waves = l.plan.waves;
        a.regs = l.plan.regs;
        a.gm_tiles = l.plan.gm_tiles;
        a.gmp = l.plan.gmp;
        a.flagged = launch_flagged(l, prob_n);
        a.partial = reinterpret_cast<float *>(ws + (a.flagged ? kCounterBytes : wl.decode_partial));
        a.group_major = g_tune.decode_group_major;
        if ((a.gmp ? launch_decode_gmp(a, st) : launch_decode(a, st)) != hipSuccess) return KILN_W4A16_ERR_LAUNCH;
    }
    return KILN_W4A16_OK;
}

}  // namespace
}  // namespace kiln

extern "C" {

size_t kiln_w4a16_workspace_bytes(int prob_m, int prob_n, int prob_k) {
    return kiln_w4a16_workspace_bytes_tuned(prob_m, prob_n, prob_k, -1, -1, -1);
}

size_t kiln_w4a16_workspace_bytes_tuned(int prob_m, int prob_n, int prob_k, int thread_k, int thread_n, int sms) {
    if (prob_n <= 0 || prob_k <= 0 || !shape_ok(prob_n, prob_k, 128)) return kZeroedBytes;
    int dev = 0;
    if (sms <= 0 && hipGetDevice(&dev) != hipSuccess) dev = -1;  // no device: the part's 256 units
    const int cus = sms > 0 ? sms : compute_units(dev);
    return workspace_bytes_upto(prob_m > 0 ? prob_m : 1, prob_n, prob_k, cus, thread_k > 0 ? thread_k : -1,
                                thread_n > 0 ? thread_n : -1);
}

size_t kiln_w4a16_workspace_zeroed_bytes(void) { return kZeroedBytes; }

// ---- the GEMM for callers that cannot hand over (or allocate) a workspace ----------------------
// The workspace of kiln_marlin_w4a16_gemm -- arrival counters and the f32 partial tiles of K-sliced
// launches -- lives in a device array of the library instead.  Each GPU the library runs on holds
// its own copy at its own address until the process ends; the loader zero-fills it, and every call
// leaves the counter prefix zero again.  In host code the array's name is only a handle: the
// address kernels may use comes from hipGetSymbolAddress, asked once per device with that device
// current, and is what every launch gets as its workspace argument.
}  // extern "C"

namespace kiln {
namespace {

constexpr size_t kStaticScratchBytes = KILN_W4A16_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

struct StaticScratch {
    std::once_flag once;
    void *ptr = nullptr;
    hipError_t err = hipErrorNotInitialized;
};
StaticScratch g_static_scratch[kMaxDevices];

// device address of the current device's copy of `scratch` (nullptr if the runtime refuses)
void *static_scratch_ptr(int current_dev) {
    StaticScratch &slot = g_static_scratch[current_dev];
    std::call_once(slot.once, [&]() {
        void *p = nullptr;
        slot.err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (slot.err == hipSuccess) slot.ptr = p;
    });
    return slot.err == hipSuccess ? slot.ptr : nullptr;
}

}  // namespace
}  // namespace kiln

extern "C" {

kiln_marlin_status_t kiln_marlin_w4a16_gemm_static_scratch(const void *A, const void *B, void *C, void *s,
                                                           int prob_m, int prob_n, int prob_k, int groupsize,
                                                           int dev, void *stream) {
    if (prob_m < 0 || prob_n < 0 || prob_k < 0) return KILN_W4A16_ERR_PROB_SHAPE;
    if (!shape_ok(prob_n, prob_k, groupsize)) return KILN_W4A16_ERR_PROB_SHAPE;
    if (prob_m == 0 || prob_n == 0 || prob_k == 0) return KILN_W4A16_OK;
    if (!A || !B || !C || !s) return KILN_W4A16_ERR_ARGUMENT;
    // the array belongs to the device that is current: that must be the one the caller names
    int current = -1;
    if (hipGetDevice(&current) != hipSuccess || current != dev || dev < 0 || dev >= kMaxDevices)
        return KILN_W4A16_ERR_ARGUMENT;
    GemmPlan gp;
    plan_gemm(prob_m, prob_n, prob_k, compute_units(dev), -1, -1, false, &gp);
    if (workspace_layout(gp, prob_m, prob_n, prob_k).plain > kStaticScratchBytes) return KILN_W4A16_ERR_SCRATCH;
    void *ws = static_scratch_ptr(current);
    if (!ws) return KILN_W4A16_ERR_LAUNCH;
    return gemm_any(A, B, C, s, prob_m, prob_n, prob_k, ws, groupsize, dev, stream, -1, -1, -1, nullptr);
}

kiln_marlin_status_t kiln_marlin_w4a16_gemm(const void *A, const void *B, void *C, void *s,
                                            int prob_m, int prob_n, int prob_k, void *workspace,
                                            int groupsize, int dev, void *stream, int thread_k,
                                            int thread_n, int sms, int max_par) {
    (void)max_par;
    return gemm_any(A, B, C, s, prob_m, prob_n, prob_k, workspace, groupsize, dev, stream, thread_k, thread_n, sms,
                    nullptr);
}

// ---- the sticky word of the bounded waits ---------------------------------------------------------
// workspace == nullptr: the current device's static array (kiln_marlin_w4a16_gemm_static_scratch).
static char *workspace_or_static(const void *workspace) {
    if (workspace) return reinterpret_cast<char *>(const_cast<void *>(workspace));
    int current = -1;
    if (hipGetDevice(&current) != hipSuccess || current < 0 || current >= kMaxDevices) return nullptr;
    return reinterpret_cast<char *>(static_scratch_ptr(current));
}

size_t kiln_w4a16_workspace_error_offset(void) { return kWsErrorOffset; }

kiln_marlin_status_t kiln_w4a16_workspace_check(const void *workspace, uint32_t *host_word, void *stream) {
    if (!host_word) return KILN_W4A16_ERR_ARGUMENT;
    const char *ws = workspace_or_static(workspace);
    if (!ws) return KILN_W4A16_ERR_ARGUMENT;
    return hipMemcpyAsync(host_word, ws + kWsErrorOffset, sizeof(uint32_t), hipMemcpyDeviceToHost,
                          reinterpret_cast<hipStream_t>(stream)) == hipSuccess ? KILN_W4A16_OK : KILN_W4A16_ERR_LAUNCH;
}

kiln_marlin_status_t kiln_w4a16_workspace_reset(void *workspace, void *stream) {
    char *ws = workspace_or_static(workspace);
    if (!ws) return KILN_W4A16_ERR_ARGUMENT;
    if (reinterpret_cast<uintptr_t>(ws) % 16 != 0) return KILN_W4A16_ERR_ARGUMENT;
    zero_fill_kernel<<<256, 256, 0, reinterpret_cast<hipStream_t>(stream)>>>(reinterpret_cast<u32x4 *>(ws), kZeroedBytes / 16);
    return hipGetLastError() == hipSuccess ? KILN_W4A16_OK : KILN_W4A16_ERR_LAUNCH;
}

// The small-M plan for a run of m rows on a part with `cus` compute units (a pure query, no GPU
// needed): out = {KS, GS, U, BPS, waves, direct, regs, gm_tiles}.
// m <= 32; returns 0, or 1 if no plan fits.
int kiln_w4a16_debug_decode_plan(int m, int n, int k, int cus, int *out) {
    if (m < 1 || m > 32 || cus < 1 || !shape_ok(n, k, 128)) return 1;
    const SlabChoice c = slab_choice(m, n, k, cus, -1, -1, false);
    if (!c.ok) return 1;
    const DecodePlan &p = c.plan;
    out[0] = p.KS; out[1] = p.GS; out[2] = p.U; out[3] = p.BPS; out[4] = p.waves;
    out[5] = c.direct;
    out[6] = p.regs;
    out[7] = p.gmp ? -p.gm_tiles : p.gm_tiles;   // negative: the private-staging instance
    return 0;
}

// Which path a plain GEMM takes (a pure query):
// out = {matrix-core path?, small-M launches, block rows, block columns, whole column blocks, K slices,
//        mid-M kernel?, its tile pairs * 16 + K slices}.
int kiln_w4a16_debug_gemm_plan(int m, int n, int k, int cus, int *out) {
    if (m < 1 || cus < 1 || !shape_ok(n, k, 128)) return 1;
    GemmPlan gp;
    plan_gemm(m, n, k, cus, -1, -1, false, &gp);
    out[0] = gp.prefill; out[1] = gp.launches; out[2] = gp.pf.bm; out[3] = gp.pf.bn; out[4] = gp.pf.nb_full;
    out[5] = gp.pf.ks;
    out[6] = gp.mid;          // the mid-M kernel: pairs of tiles per block, K slices
    out[7] = gp.mid ? gp.mp.pairs * 16 + gp.mp.KS : 0;
    return 0;
}

// Where the matrix-core kernel's row sums come from on a plain GEMM of these sizes: > 0 = that many blocks
// of its own launch, 0 = a launch in front, -2 = every block sums its own rows, -3 = another kernel runs;
// -1 = bad sizes
int kiln_w4a16_debug_prefill_rowsum_producers(int m, int n, int k, int cus) {
    if (m < 1 || cus < 1 || !shape_ok(n, k, 128)) return -1;
    GemmPlan gp;
    plan_gemm(m, n, k, cus, -1, -1, false, &gp);
    if (!gp.prefill) return -3;
    const int inside = prefill_rowsum_producers(m, n, k, gp.pf, cus);
    return inside > 0 && g_tune.rowsum_fold == 0 ? 0 : inside;
}

#ifdef KILN_W4A16_TUNING_HOOKS
// Only in the tuning build of the library (never in the shipped one): process-wide overrides of
// the automatic plan for the test suite and profiling scripts (0 / -1 = automatic).  Plain
// globals: set them only while no other thread is inside a GEMM call.
static void tuning_changed() {
    std::lock_guard<std::mutex> lock(g_plan_mutex);
    g_plan_cache.clear();
}
void kiln_w4a16_debug_prefill_min_m(int m) { g_tune.prefill_min_m = m > 0 ? m : 0; tuning_changed(); }
void kiln_w4a16_debug_prefill_ks(int ks) { g_tune.prefill_ks = ks; }
void kiln_w4a16_debug_prefill_bn(int bn) { g_tune.prefill_bn = bn; }
void kiln_w4a16_debug_prefill_bm(int bm) { g_tune.prefill_bm = bm; }
void kiln_w4a16_debug_prefill_nb_full(int nb) { g_tune.prefill_nb_full = nb; }
void kiln_w4a16_debug_decode_direct_max_m(int m) { g_tune.decode_direct_max_m = m; tuning_changed(); }
void kiln_w4a16_debug_decode_group_major(int mode) { g_tune.decode_group_major = mode; tuning_changed(); }
void kiln_w4a16_debug_decode_runs_per_launch(int runs) { g_tune.decode_runs_per_launch = runs; }
void kiln_w4a16_debug_gmp(int tiles, int waves, int kslices) {
    g_tune.gmp_tiles = tiles;
    g_tune.gmp_waves = waves;
    g_tune.gmp_ks = kslices;
    tuning_changed();
}
void kiln_w4a16_debug_flagged(int mode) { g_tune.flagged = mode; tuning_changed(); }
void kiln_w4a16_debug_lora_fold(int mode) { g_tune.lora_fold = mode; }
void kiln_w4a16_debug_rowsum_fold(int mode) { g_tune.rowsum_fold = mode; }
void kiln_w4a16_debug_mid(int mode, int pairs, int kslices) {
    g_tune.mid = mode;
    g_tune.mid_pairs = pairs;
    g_tune.mid_ks = kslices;
}
void kiln_w4a16_debug_mid_waves(int waves) { g_tune.mid_waves = waves > 0 ? waves : 0; }
void kiln_w4a16_debug_tune(int waves, int run, int kslices) {
    g_tune.force_waves = waves;
    g_tune.force_u = run;
    g_tune.force_ks = kslices;
    tuning_changed();
}
#endif

kiln_marlin_status_t kiln_w4a16_dequant_f32(const void *B, const void *s, int prob_k, int prob_n,
                                            int groupsize, void *out, int dev, void *stream) {
    (void)dev;
    if (prob_k < 0 || prob_n < 0 || !shape_ok(prob_n, prob_k, groupsize)) return KILN_W4A16_ERR_PROB_SHAPE;
    if (prob_k == 0 || prob_n == 0) return KILN_W4A16_OK;
    if (!B || !s || !out) return KILN_W4A16_ERR_ARGUMENT;
    const int G = prob_k / kGroupK;
    const int chunks = (prob_n / kTileN) * G;
    dequant_f32_kernel<<<chunks, 64, 0, reinterpret_cast<hipStream_t>(stream)>>>(
        (const u32x4 *)B, (const uint16_t *)s, (float *)out, prob_k, prob_n,
        groupsize == -1 ? 1 : G);
    return hipGetLastError() == hipSuccess ? KILN_W4A16_OK : KILN_W4A16_ERR_LAUNCH;
}

kiln_marlin_status_t kiln_w4a16_gemm_lora(const void *A, const void *B, void *C, const void *s,
                                          int prob_m, int prob_n, int prob_k, void *workspace,
                                          int groupsize, int dev, void *stream, const void *lora_a,
                                          const void *lora_b, int r_total, int n_adapters,
                                          const int *ranks, const float *scales) {
    if (prob_m < 0 || prob_n < 0 || prob_k < 0) return KILN_W4A16_ERR_PROB_SHAPE;
    if (!shape_ok(prob_n, prob_k, groupsize)) return KILN_W4A16_ERR_PROB_SHAPE;
    if (r_total < 1 || n_adapters < 1 || !ranks || !scales) return KILN_W4A16_ERR_ARGUMENT;
    if (r_total > 64 || n_adapters > 8) return KILN_W4A16_ERR_KERN_SHAPE;
    int sum = 0;
    for (int i = 0; i < n_adapters; ++i) {
        if (ranks[i] < 1) return KILN_W4A16_ERR_ARGUMENT;
        sum += ranks[i];
    }
    if (sum != r_total) return KILN_W4A16_ERR_ARGUMENT;
    if (prob_m == 0 || prob_n == 0 || prob_k == 0) return KILN_W4A16_OK;
    if (!A || !B || !C || !s || !workspace || !lora_a || !lora_b) return KILN_W4A16_ERR_ARGUMENT;
    if (reinterpret_cast<uintptr_t>(lora_a) % 16 != 0 || reinterpret_cast<uintptr_t>(lora_b) % 16 != 0) return KILN_W4A16_ERR_ARGUMENT;

    const LoraSpec lora{lora_a, lora_b, r_total, n_adapters, ranks, scales};
    return gemm_any(A, B, C, s, prob_m, prob_n, prob_k, workspace, groupsize, dev, stream, -1, -1, -1, &lora);
}

kiln_marlin_status_t kiln_w4a16_gemm_swiglu(const void *A, const void *B, void *C, const void *s,
                                            int prob_m, int n_out, int prob_k, void *workspace,
                                            int groupsize, int dev, void *stream) {
    if (prob_m < 0 || n_out < 0 || prob_k < 0 || n_out > INT32_MAX / 2) return KILN_W4A16_ERR_PROB_SHAPE;
    // packed columns: per 16-column tile 8 gate columns, then the 8 matching up columns; every kernel
    // forms silu(gate) * up where it stores a tile, from the f32 sums
    return gemm_any(A, B, C, s, prob_m, 2 * n_out, prob_k, workspace, groupsize, dev, stream, -1, -1, -1, nullptr, true);
}

kiln_marlin_status_t kiln_w4a16_gemm_swiglu_lora(const void *A, const void *B, void *C, const void *s, int prob_m,
                                                 int n_out, int prob_k, void *workspace, int groupsize, int dev,
                                                 void *stream, const void *lora_a, const void *lora_b, int r_total,
                                                 int n_adapters, const int *ranks, const float *scales) {
    if (prob_m < 0 || n_out < 0 || prob_k < 0 || n_out > INT32_MAX / 2) return KILN_W4A16_ERR_PROB_SHAPE;
    if (!shape_ok(2 * n_out, prob_k, groupsize)) return KILN_W4A16_ERR_PROB_SHAPE;
    if (r_total < 1 || n_adapters < 1 || !ranks || !scales) return KILN_W4A16_ERR_ARGUMENT;
    if (r_total > 64 || n_adapters > 8) return KILN_W4A16_ERR_KERN_SHAPE;
    int sum = 0;
    for (int i = 0; i < n_adapters; ++i) {
        if (ranks[i] < 1) return KILN_W4A16_ERR_ARGUMENT;
        sum += ranks[i];
    }
    if (sum != r_total) return KILN_W4A16_ERR_ARGUMENT;
    if (prob_m == 0 || n_out == 0 || prob_k == 0) return KILN_W4A16_OK;
    if (!A || !B || !C || !s || !workspace || !lora_a || !lora_b) return KILN_W4A16_ERR_ARGUMENT;
    if (reinterpret_cast<uintptr_t>(lora_a) % 16 != 0 || reinterpret_cast<uintptr_t>(lora_b) % 16 != 0) return KILN_W4A16_ERR_ARGUMENT;
    // the low-rank term lands on the f32 sums of gate and up before silu(gate) * up is formed; lora_b's rows
    // follow the packed columns, so an adapter of gate and one of up are two column blocks of one stacked B
    const LoraSpec lora{lora_a, lora_b, r_total, n_adapters, ranks, scales};
    return gemm_any(A, B, C, s, prob_m, 2 * n_out, prob_k, workspace, groupsize, dev, stream, -1, -1, -1, &lora, true);
}

// ---- the MLP of a layer as one call -------------------------------------------------------------------
// workspace: [what the two GEMMs need, the larger of the two] | H = bf16 [m, n_out]
static size_t mlp_h_offset(int m, int k1, int n_out, int n2) {
    const size_t a = kiln_w4a16_swiglu_workspace_bytes(m, n_out, k1), b = kiln_w4a16_workspace_bytes(m, n2, n_out);
    return ((a > b ? a : b) + 255) & ~(size_t)255;
}

size_t kiln_w4a16_mlp_workspace_bytes(int prob_m, int hidden, int n_out, int n_down) {
    if (prob_m < 1) prob_m = 1;
    if (hidden <= 0 || n_out <= 0 || n_down <= 0 || n_out > INT32_MAX / 2) return kZeroedBytes;
    return mlp_h_offset(prob_m, hidden, n_out, n_down) + (size_t)prob_m * n_out * 2;
}

kiln_marlin_status_t kiln_w4a16_mlp(const void *x, const void *b_gate_up, const void *s_gate_up, const void *b_down,
                                    const void *s_down, void *y, int prob_m, int hidden, int n_out, int n_down,
                                    void *workspace, int groupsize, int dev, void *stream) {
    if (prob_m < 0 || hidden < 0 || n_out < 0 || n_down < 0 || n_out > INT32_MAX / 2) return KILN_W4A16_ERR_PROB_SHAPE;
    if (!shape_ok(2 * n_out, hidden, groupsize) || !shape_ok(n_down, n_out, groupsize)) return KILN_W4A16_ERR_PROB_SHAPE;
    if (prob_m == 0 || hidden == 0 || n_out == 0 || n_down == 0) return KILN_W4A16_OK;
    if (!x || !b_gate_up || !s_gate_up || !b_down || !s_down || !y || !workspace) return KILN_W4A16_ERR_ARGUMENT;
    char *ws = reinterpret_cast<char *>(workspace);
    void *h = ws + mlp_h_offset(prob_m, hidden, n_out, n_down);
    // Two launches with H in between.  (One launch for both -- down blocks resident from the start, their weights
    // in registers, waiting for their columns of H -- measured level with the two, 15.2 us at 16 rows: every hop
    // of the hand-over inside a launch crosses the dies' memory system, about a microsecond each.)
    const kiln_marlin_status_t st = gemm_any(x, b_gate_up, h, s_gate_up, prob_m, 2 * n_out, hidden, workspace, groupsize, dev,
                                             stream, -1, -1, -1, nullptr, true);
    if (st != KILN_W4A16_OK) return st;
    return gemm_any(h, b_down, y, s_down, prob_m, n_down, n_out, workspace, groupsize, dev, stream, -1, -1, -1, nullptr);
}

size_t kiln_w4a16_swiglu_workspace_bytes(int prob_m, int n_out, int prob_k) {
    if (n_out <= 0 || n_out > INT32_MAX / 2) return kZeroedBytes;
    return kiln_w4a16_workspace_bytes(prob_m, 2 * n_out, prob_k);  // the same plans as the plain GEMM of that width
}

}  // extern "C"
