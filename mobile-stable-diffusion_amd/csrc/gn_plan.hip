// Launch plan of the GroupNorm register kernels (host arithmetic, no device code).
//
// A plan is (slices per unit, lanes per workgroup, 16-byte vectors per lane, writers per whole
// unit).  It comes from three places, in this order:
//   1. the tuning knobs, when a test or a sweep forces a value;
//   2. a table of measured plans (gn_plan_table.inc) for the shapes the library is tuned for:
//      an exact match on (element size, vectors per unit, units, output apart from the input),
//      used on the chip the table was measured on only (256 CUs in 8 XCDs);
//   3. a rule that needs nothing but the chip's CU / XCD count and a few constants: how many
//      workgroups the launch has per CU decides whether one workgroup's latency or the chip's
//      throughput is what to plan for.
// `bench.py --tables gn_plan_sweep` times the result against every plan the knobs can force,
// with and without the table; gn_plan_table.py writes the table from such a sweep.
#include <algorithm>

#include "msd_device.h"
#include "msd_internal.h"

namespace msd {

namespace {

// ---- what the kernels are built for ------------------------------------------------------
const int kKValues[] = {1, 2, 3, 4, 5, 6, 8, 10, 12, 16, 20};

inline int round_up_k(uint32_t k) {
    for (int v : kKValues)
        if ((uint32_t)v >= k) return v;
    return 0;
}

// Wavefronts of gn_slice_kernel<T, K> a SIMD holds at once: eight slots, fewer when the
// instance's registers do not allow eight (512 per lane and SIMD; K <= 8 needs at most 64,
// K = 10 / 12 / 16 / 20 need 74 / 85 / 120 / 121 - the compiler's resource report).
inline uint32_t waves_per_simd(int k) { return k <= 8 ? 8u : k == 10 ? 6u : k == 12 ? 5u : 4u; }

// All `blocks` workgroups of `threads` lanes are on the chip at once: a workgroup puts a quarter of
// its wavefronts (rounded up) on each of a CU's four SIMDs.
inline bool launch_is_resident(const Chip &chip, size_t blocks, uint32_t threads, int k) {
    const uint32_t per_simd = (threads / kWave + 3) / 4;
    return blocks <= (size_t)chip.cus * (waves_per_simd(k) / per_simd);
}

// Relative cost of holding a slice as K vectors per lane when a workgroup has a CU to itself
// (measured on whole units of 1280 ... 15360 vectors, one workgroup per CU, against the best
// size for the same unit): 1, 2, 3, 5 cost nothing, 10 and 20 little, 4 / 6 / 8 / 12 / 16 lose
// 3 - 8 % (longer dependent chains for the same number of wavefronts).
inline float k_cost(int k) {
    switch (k) {
        case 4: return 0.03f;
        case 6: case 8: return 0.06f;
        case 10: return 0.02f;
        case 12: return 0.08f;
        case 16: return 0.05f;
        case 20: return 0.03f;
        default: return 0.0f;
    }
}

// A workgroup normalises about this many elements in the time an exchange between the slices of
// a unit costs (two round trips through the memory-side coherence point, 1.3 - 2.5 us): units up
// to this size stay whole, longer ones are cut into slices of at most this size.  In elements,
// not bytes: the epilogue's arithmetic per element is what a slice's time is made of.
constexpr size_t kSliceElements = 20480;
constexpr size_t kMinSliceVectors = 960;  // no slice is made shorter than this to fill idle CUs

inline uint32_t round_up_wave(size_t n) { return (uint32_t)(((n + kWave - 1) / kWave) * kWave); }

// One row of the table of measured plans.
struct GnTunedPlan {
    uint8_t elt;        // bytes per element
    uint8_t apart;      // 1: output apart from the input (units may be shared), 0: in place
    uint32_t vectors;   // 16-byte vectors per unit
    uint32_t units;     // batch * groups
    uint8_t split;
    uint16_t threads;
    uint8_t writers;
};

const GnTunedPlan kTunedPlans[] = {
#include "gn_plan_table.inc"
    {0, 0, 0, 0, 0, 0, 0},  // (end: matches no shape)
};

const GnTunedPlan *tuned_plan(size_t elt, size_t vectors, size_t units, bool apart) {
    for (const GnTunedPlan &row : kTunedPlans)
        if (row.elt == elt && row.vectors == vectors && row.units == units && (row.apart != 0) == apart) return &row;
    return nullptr;
}

}  // namespace

// K for a slice of `vecs` vectors on `threads` lanes, 0 if there is none.  The largest K has
// no code for a ragged slice: it takes equal slices that it fits exactly.
int gn_k_for(uint32_t vecs, uint32_t threads, uint32_t max_k, bool equal_slices) {
    const int k = round_up_k((vecs + threads - 1) / threads);
    if (k == 0 || (uint32_t)k > max_k) return 0;
    if (k == kGnMaxK && !(equal_slices && vecs == (uint32_t)k * threads)) return 0;
    return k;
}

// The chip the current device is: compute units and XCDs (the dispatcher deals consecutive
// workgroups to the XCDs in turn; each XCD has an L2 of its own).  Asked once per device; the
// knobs MSD_TUNE_DEVICE_CUS / _XCDS replace the answer (tests plan for other chips with them);
// without a device (planning on a host that has none) the MI355X's 256 CUs in 8 XCDs.
Chip chip_info() {
    constexpr int kMaxDevices = 64;
    static std::atomic<uint32_t> cached[kMaxDevices];  // (cus << 8) | xcds, 0 = not asked yet
    Chip chip{256, 8};
    int device = 0;
    if (hipGetDevice(&device) == hipSuccess && device >= 0 && device < kMaxDevices) {
        uint32_t packed = cached[device].load(std::memory_order_relaxed);
        if (packed == 0) {
            int cus = 0, xcds = 0;
            if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && cus > 0) {
                if (hipDeviceGetAttribute(&xcds, hipDeviceAttributeNumberOfXccs, device) != hipSuccess || xcds <= 0) xcds = 1;
                packed = ((uint32_t)cus << 8) | (uint32_t)std::min(xcds, 255);
                cached[device].store(packed, std::memory_order_relaxed);
            }
        }
        if (packed != 0) chip = Chip{packed >> 8, packed & 255u};
    } else {
        (void)hipGetLastError();  // no device: not an error of the caller's
    }
    const int tune_cus = g_tuning.device_cus.load(std::memory_order_relaxed);
    const int tune_xcds = g_tuning.device_xcds.load(std::memory_order_relaxed);
    if (tune_cus > 0) chip.cus = (uint32_t)tune_cus;
    if (tune_xcds > 0) chip.xcds = (uint32_t)tune_xcds;
    return chip;
}

// Writers per whole unit when the launch may share units (1: it does not).  A unit's time is
// its load, its statistics and the epilogue of SiLU and stores, one behind the other on one
// CU; with w workgroups per unit, each loading and reducing all of it (the copies meet in the
// L2 of the XCD they share) and finishing a w-th of it, the epilogue and the stores shrink to
// a w-th while nothing is exchanged.  w = as many as give the chip one workgroup per CU, 8 at
// most.  Past 5120 vectors of 2-byte elements (10240 of 4-byte ones, 5120 with eight writers)
// the repeated loads cost more than the shorter epilogue gains.
uint32_t gn_auto_writers(const Chip &chip, size_t elt, size_t units, size_t vec_per_unit) {
    // The writers of a unit must run on one XCD (block ids a multiple of the XCD count apart),
    // which needs a power-of-two XCD count and the units in whole rows of that many; on
    // different XCDs every copy of the loads comes from memory and the launch is slower than
    // with one writer.
    if ((chip.xcds & (chip.xcds - 1)) != 0 || units % chip.xcds != 0) return 1;
    uint32_t w = 1;
    while (w < 8 && units * w * 2 <= chip.cus) w *= 2;
    const size_t limit = (elt == 2 || w >= 8) ? 5120 : 10240;
    return vec_per_unit <= limit ? w : 1;
}

// Lanes and K for a workgroup that holds `vecs` vectors in a launch of `blocks` workgroups.
// `split`: slices per unit of the launch; `shared`: every workgroup holds a whole unit that
// several of them finish.
GnThreads gn_threads_for(const Chip &chip, size_t elt, uint32_t vecs, uint32_t split, size_t blocks, uint32_t max_k,
                         bool equal_slices, bool shared) {
    GnThreads pl{0, 0};
    auto k_of = [&](uint32_t t) { return gn_k_for(vecs, t, max_k, equal_slices); };
    if (blocks > chip.cus) {
        // Throughput: the CUs hold several workgroups each, in different phases (load, statistics,
        // store).  The smallest of 256 ... 1024 lanes that holds the unit (512 ... for slices of cut
        // units) - fewer, longer wavefronts, a barrier that joins four of them instead of sixteen,
        // and the whole launch resident at once (K = 20 on 256 lanes: four wavefronts per
        // workgroup, four per SIMD) - as long as short units still give every CU ten wavefronts to
        // hide latency with.  From eight workgroups per CU on, slices of cut units take the
        // smallest workgroup that holds them in at most five vectors per lane instead (eight
        // wavefronts per SIMD).
        if (split > 1 && blocks >= 8 * (size_t)chip.cus)
            for (uint32_t t = 256; t <= kGnMaxThreads && pl.threads == 0; t += kWave) {
                const int k = k_of(t);
                if (k != 0 && k <= 5) pl.threads = t;
            }
        uint32_t smallest = 0;
        for (uint32_t t = 256; t <= kGnMaxThreads && pl.threads == 0; t += 256) {
            if (k_of(t) == 0 || (split > 1 && t == 256)) continue;
            if (smallest == 0) smallest = t;
            if (vecs <= 4096 && blocks * (t / kWave) < 10 * (size_t)chip.cus && t < kGnMaxThreads) continue;
            pl.threads = t;
        }
        if (pl.threads == 0) pl.threads = kGnMaxThreads;
        // (more wavefronts per CU are not worth a launch that no longer fits the chip at once)
        if (smallest != 0 && smallest != pl.threads && k_of(pl.threads) != 0 &&
            !launch_is_resident(chip, blocks, pl.threads, k_of(pl.threads)) &&
            launch_is_resident(chip, blocks, smallest, k_of(smallest)))
            pl.threads = smallest;
    } else if (shared && vecs <= 2560) {
        // every writer reduces the whole unit and a part of its wavefronts does the epilogue:
        // fewer lanes with more vectors each than a lone workgroup would take
        pl.threads = (vecs == 2560) ? 640u : vecs > 704 ? 512u : vecs >= 256 ? 384u : round_up_wave(vecs);
    } else if (vecs <= 704) {
        pl.threads = round_up_wave(vecs);  // one vector per lane
    } else if (shared && k_of(kGnMaxThreads) != 0 && k_of(kGnMaxThreads) <= 5) {
        pl.threads = kGnMaxThreads;
    } else {
        // Latency: the workgroup has a CU to itself.  512 ... 1024 lanes; the size whose K costs
        // least, then the one with the fewest masked lanes, then the larger.
        float best = 1e9f;
        for (uint32_t t = 512; t <= kGnMaxThreads; t += kWave) {
            const int k = k_of(t);
            if (k == 0) continue;
            const float cost = k_cost(k) + 0.02f * (float)((size_t)k * t - vecs) / (float)vecs - 0.001f * (float)t / 1024.0f;
            if (cost < best - 1e-6f) {
                best = cost;
                pl.threads = t;
            }
        }
        if (pl.threads == 0) pl.threads = kGnMaxThreads;
    }
    pl.k = k_of(pl.threads);
    return pl;
}

namespace {

// Slices per unit the rule wants for whole units of `vec_per_unit` vectors (1: whole).
uint32_t rule_split(const Chip &chip, size_t elt, size_t units, size_t vec_per_unit) {
    const size_t epv = 16 / elt;
    const size_t slice = kSliceElements / epv;  // vectors
    uint32_t want = 1;
    if (units < chip.cus) {
        // Latency: fewer units than CUs.  (4-byte elements at less than a quarter of the chip:
        // units stay whole up to four fifths of the usual size.)
        const size_t whole = (elt == 2 || units * 4 >= chip.cus) ? slice : slice * 4 / 5;
        // ... cut while every workgroup still gets a CU of its own (two per CU for 4-byte elements:
        // half the arithmetic per vector): in two, then halved until a slice is at most that size
        const size_t cap = elt == 2 ? chip.cus : 2 * (size_t)chip.cus;
        if (vec_per_unit > whole && units * 2 <= cap) {
            want = 2;
            while (vec_per_unit > want * slice && units * want * 2 <= cap && want < 8) want *= 2;
            // ... and on, down to slices of 960 vectors, while less than half of the CUs have one
            while (units * want * 2 < chip.cus && vec_per_unit / (want * 2) >= kMinSliceVectors && want < 8) want *= 2;
        }
    } else if (elt == 4 && units < 2 * (size_t)chip.cus) {
        if (vec_per_unit > slice) want = 2;  // one to two units per CU, 4-byte elements: halves
    } else if (units >= 2 * (size_t)chip.cus && vec_per_unit > 10240) {
        // Throughput, very long units: slices of at most 2560 vectors on small workgroups overlap
        // better than whole units on 768 - 1024 lanes; the exchange disappears behind the other
        // workgroups of the CU.
        while (vec_per_unit > (size_t)want * 2560 && want < 8) want *= 2;
    }
    // Between one and two workgroups per CU a launch runs as two rounds with the second mostly
    // empty.  Slices of units shorter than three times the size above are merged back (a CU each,
    // or nearly); longer units, and whole units from twice that size on, are cut once more (two
    // and more workgroups on every CU).
    const size_t blocks = units * want;
    if (blocks > chip.cus && blocks < 2 * (size_t)chip.cus) {
        if (want > 1 && vec_per_unit < 3 * slice)
            want /= 2;
        else if (vec_per_unit >= 2 * slice && want < 8)
            want *= 2;
    }
    while (units * want < 16 && want < kGnMaxSplit) want *= 2;  // very few units
    return want;
}

}  // namespace

// What a GroupNorm launch looks like for a shape: split == 0 means the general kernel (one
// workgroup per unit, any alignment); otherwise `split` workgroups of `threads` lanes per unit,
// each holding its slice as `k` vectors per lane.  `elt` = bytes per element, `max_units` = units
// the exchange scratch has room for.  `writers` > 1 (only where `may_share`: the output does
// not overlap the input) means whole units with that many workgroups each, every one loading and
// reducing the whole unit and storing its part of it.  Reads the tuning knobs.
GnDecision gn_decide(size_t elt, size_t batch, size_t channels, size_t hw, size_t groups, bool aligned,
                     size_t max_units, bool may_share) {
    GnDecision d{0, 0, 0, 0, 1};
    const size_t epv = 16 / elt;
    const size_t cpg = channels / groups;
    const size_t unit_size = cpg * hw;
    const size_t units = batch * groups;
    // (the register kernel addresses a unit with 32-bit byte offsets)
    if (!aligned || hw % epv != 0 || unit_size * elt >= (1ull << 32)) return d;
    const size_t vec_per_unit = unit_size / epv;
    const Chip chip = chip_info();

    const int tune_split = g_tuning.gn_split.load(std::memory_order_relaxed);
    const int tune_threads = g_tuning.gn_threads.load(std::memory_order_relaxed);
    const int tune_writers = g_tuning.gn_writers.load(std::memory_order_relaxed);
    const bool rule_only = g_tuning.gn_plan_rule_only.load(std::memory_order_relaxed) != 0;
    const bool can_split = units <= max_units;
    // gamma / beta of the group go through LDS from seven vectors per lane on
    auto affine_fits = [&](int k) { return !(k > kGnPrefetchAffineK && cpg > kGnLdsChannels); };

    // ---- a measured plan for exactly this shape, on the chip it was measured on.  (With the
    // writers knob at 1, "never share", a launch whose output lies apart is planned exactly like
    // the call in place: tests compare the two bit for bit.)
    if (tune_writers == 1) may_share = false;
    const GnTunedPlan *tuned = nullptr;
    if (tune_split == 0 && tune_threads == 0 && tune_writers <= 1 && !rule_only && chip.cus == 256 && chip.xcds == 8)
        tuned = tuned_plan(elt, vec_per_unit, units, may_share);

    // ---- several writers per whole unit
    if (may_share && tune_split <= 1 && vec_per_unit <= (size_t)kGnMaxThreads * kGnSharedMaxK &&
        (tuned == nullptr || tuned->writers > 1)) {
        uint32_t writers = tuned ? tuned->writers
                           : tune_writers > 1 ? (uint32_t)tune_writers
                                              : gn_auto_writers(chip, elt, units, vec_per_unit);
        while (writers > 1 && vec_per_unit < (size_t)writers * kWave) writers /= 2;  // a part is at least a wavefront's vectors
        if (units * writers > 0x7FFFFFFFull) writers = 1;                            // (the grid is units * writers blocks)
        if (writers > 1) {
            GnThreads pl{0, 0};
            uint32_t force = tuned ? tuned->threads : 0;
            if (tune_threads >= kWave && tune_threads <= kGnMaxThreads && tune_threads % kWave == 0) force = (uint32_t)tune_threads;
            if (force != 0 && gn_k_for((uint32_t)vec_per_unit, force, kGnSharedMaxK, true) != 0)
                pl = GnThreads{force, gn_k_for((uint32_t)vec_per_unit, force, kGnSharedMaxK, true)};
            else
                pl = gn_threads_for(chip, elt, (uint32_t)vec_per_unit, 1, units * writers, kGnSharedMaxK, true, true);
            if (pl.k != 0 && affine_fits(pl.k)) {
                d.split = 1;
                d.threads = pl.threads;
                d.k = (uint32_t)pl.k;
                d.vec_per_slice = (uint32_t)vec_per_unit;
                d.writers = writers;
                return d;
            }
        }
    }

    // ---- slices: the smallest power-of-two count whose slices fit in registers, then what the
    // knob, the table or the rule asks for
    const size_t slice_cap = (size_t)kGnMaxThreads * kGnMaxRaggedK;  // vectors one workgroup can hold
    uint32_t split = 1;
    while ((size_t)split * slice_cap < vec_per_unit && split <= kGnMaxSplit) split *= 2;
    if (split > kGnMaxSplit || (split > 1 && !can_split)) return d;
    if (tune_split > 0) {
        const uint32_t forced = (uint32_t)tune_split;
        if (forced > split && can_split && (forced & (forced - 1)) == 0 && forced <= kGnMaxSplit &&
            vec_per_unit >= (size_t)forced * kWave)
            split = forced;
    } else if (can_split) {
        const uint32_t want = (tuned && tuned->writers <= 1) ? tuned->split : rule_split(chip, elt, units, vec_per_unit);
        while (split < want && vec_per_unit >= (size_t)2 * split * 256) split *= 2;
    }

    const size_t vec_per_slice = (vec_per_unit + split - 1) / split;
    // every slice must own at least one vector (ceil division can starve the last ones)
    if (vec_per_slice * (split - 1) >= vec_per_unit) return d;
    const bool equal_slices = vec_per_slice * split == vec_per_unit;

    GnThreads pl{0, 0};
    uint32_t force = (tuned && tuned->writers <= 1 && tuned->split == split) ? tuned->threads : 0;
    if (tune_threads >= kWave && tune_threads <= kGnMaxThreads && tune_threads % kWave == 0) force = (uint32_t)tune_threads;
    if (force != 0 && gn_k_for((uint32_t)vec_per_slice, force, kGnMaxK, equal_slices) != 0)
        pl = GnThreads{force, gn_k_for((uint32_t)vec_per_slice, force, kGnMaxK, equal_slices)};
    else
        pl = gn_threads_for(chip, elt, (uint32_t)vec_per_slice, split, units * split, kGnMaxK, equal_slices, false);
    if (pl.k == 0 || !affine_fits(pl.k)) return d;
    d.split = split;
    d.threads = pl.threads;
    d.k = (uint32_t)pl.k;
    d.vec_per_slice = (uint32_t)vec_per_slice;
    return d;
}

}  // namespace msd
