// Device memory sorted by where it lies in HBM.  No counterpart in the reference (its extension leaves
// placement to torch's allocator, reference cuda/bindings.cu:98,144,183).
//
// The 288 GiB of an MI355X behave as three regions of 96 GiB: a kernel that reads one region and writes
// another moves 8-12 % more bytes per second than one that reads and writes inside one region (a flat
// copy: 5.7-6.1 TB/s inside, 6.3-6.5 TB/s across; reads alone and writes alone do not care).  Which
// region an allocation lands in is the driver's choice, and after a few processes have come and gone
// it no longer follows the order of the requests.  So this file does not guess: it takes physical
// memory in chunks (hipMemCreate), finds out by timed copies which chunks disturb each other, and maps
// chunks of one kind behind each other into three address ranges ("arenas").  What is left over goes
// back to the driver.  The host side (sinabs/exodus/hbm.py) hands out tensors from the arenas.
//
//   exodus_hbm_regions_create(device, bytes_per_region, chunk_bytes, &report)
//   exodus_hbm_regions_destroy(device)
//
// Both calls synchronise the device.  One set of arenas per device; creating a second one fails with
// hipErrorInvalidValue until the first is destroyed.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>
#include <mutex>
#include <vector>

#include "exodus_common.hpp"
#include "exodus_hip.h"

#define EXODUS_API __attribute__((visibility("default")))

namespace {

constexpr int REGIONS = EXODUS_HBM_REGIONS;
constexpr int MAX_DEVICES = 64;
constexpr int PROBES = EXODUS_HBM_PROBES;   // chunks whose pairwise copy rates are measured to find the kinds
constexpr int COPY_PER_THREAD = 4;

__global__ void __launch_bounds__(256) region_copy(f32x4 *__restrict__ dst, const f32x4 *__restrict__ src,
                                                   const int64_t n_chunks)
{
    const int64_t base = (static_cast<int64_t>(blockIdx.x) * COPY_PER_THREAD) * 256 + threadIdx.x;
    f32x4 v[COPY_PER_THREAD];
#pragma unroll
    for (int k = 0; k < COPY_PER_THREAD; ++k)
        if (base + k * 256 < n_chunks) v[k] = ld_stream(src + base + k * 256);
#pragma unroll
    for (int k = 0; k < COPY_PER_THREAD; ++k)
        if (base + k * 256 < n_chunks) st_stream(v[k], dst + base + k * 256);
}

struct Arenas {
    bool live = false;
    size_t chunk = 0;
    void *base[REGIONS] = {nullptr, nullptr, nullptr};
    size_t reserved[REGIONS] = {0, 0, 0};
    std::vector<hipMemGenericAllocationHandle_t> handles[REGIONS];
};

std::mutex table_mutex;
Arenas table[MAX_DEVICES];

// everything create() holds while it sorts; the destructor gives back whatever was not moved into an arena
struct Sorting {
    size_t chunk = 0;
    char *va = nullptr;
    size_t va_bytes = 0;
    std::vector<hipMemGenericAllocationHandle_t> handle;
    std::vector<char> mapped, owned;
    hipEvent_t e0 = nullptr, e1 = nullptr;

    ~Sorting()
    {
        (void)hipDeviceSynchronize();
        for (size_t i = 0; i < handle.size(); ++i) {
            if (mapped[i]) (void)hipMemUnmap(va + i * chunk, chunk);
            if (owned[i]) (void)hipMemRelease(handle[i]);
        }
        if (va) (void)hipMemAddressFree(va, va_bytes);
        if (e0) (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
    }

    char *at(size_t i) const { return va + i * chunk; }

    // GB/s of a copy of `bytes` from src to dst: best of `reps` after one untimed run
    hipError_t rate(void *dst, const void *src, size_t bytes, int reps, float *out)
    {
        const int64_t n16 = static_cast<int64_t>(bytes / 16);
        const unsigned blocks = static_cast<unsigned>((n16 + 256 * COPY_PER_THREAD - 1) / (256 * COPY_PER_THREAD));
        float best = 0.f;
        for (int r = 0; r <= reps; ++r) {
            hipError_t e = hipEventRecord(e0, nullptr);
            if (e != hipSuccess) return e;
            hipLaunchKernelGGL(region_copy, dim3(blocks), dim3(256), 0, nullptr, static_cast<f32x4 *>(dst),
                               static_cast<const f32x4 *>(src), n16);
            if ((e = hipGetLastError()) != hipSuccess) return e;
            if ((e = hipEventRecord(e1, nullptr)) != hipSuccess) return e;
            if ((e = hipEventSynchronize(e1)) != hipSuccess) return e;
            float ms = 0.f;
            if ((e = hipEventElapsedTime(&ms, e0, e1)) != hipSuccess) return e;
            if (r > 0 && ms > 0.f) best = std::max(best, 2.f * static_cast<float>(bytes) / ms / 1e6f);
        }
        *out = best;
        return hipSuccess;
    }
};

#define HBM_TRY(call)                          \
    do {                                       \
        const hipError_t status_ = (call);     \
        if (status_ != hipSuccess) return static_cast<int>(status_); \
    } while (0)

// The rates fall into two groups (same kind of memory: slower; different kinds: faster) that overlap a
// little at their edges: the threshold is the middle between the two group means, found by moving each
// value to the nearer mean until nothing moves (two-means in one dimension).
float two_group_threshold(const std::vector<float> &v)
{
    float lo = *std::min_element(v.begin(), v.end()), hi = *std::max_element(v.begin(), v.end());
    for (int round = 0; round < 50; ++round) {
        const float mid = 0.5f * (lo + hi);
        double sum_lo = 0, sum_hi = 0;
        int n_lo = 0, n_hi = 0;
        for (float x : v) (x < mid ? (sum_lo += x, ++n_lo) : (sum_hi += x, ++n_hi));
        if (n_lo == 0 || n_hi == 0) break;
        const float new_lo = static_cast<float>(sum_lo / n_lo), new_hi = static_cast<float>(sum_hi / n_hi);
        if (new_lo == lo && new_hi == hi) break;
        lo = new_lo; hi = new_hi;
    }
    return 0.5f * (lo + hi);
}

int create(int device, uint64_t bytes_per_region, uint64_t chunk_bytes, exodus_hbm_report *rep)
{
    HBM_TRY(hipSetDevice(device));
    HBM_TRY(hipDeviceSynchronize());
    hipMemAllocationProp prop = {};
    prop.type = hipMemAllocationTypePinned;
    prop.location.type = hipMemLocationTypeDevice;
    prop.location.id = device;
    size_t gran = 0;
    HBM_TRY(hipMemGetAllocationGranularity(&gran, &prop, hipMemAllocationGranularityRecommended));
    if (gran == 0 || chunk_bytes % gran != 0 || chunk_bytes % (16 * 256 * COPY_PER_THREAD) != 0) return hipErrorInvalidValue;
    const size_t chunk = chunk_bytes;
    const size_t need = (bytes_per_region + chunk - 1) / chunk;          // chunks per arena
    size_t free_b = 0, total_b = 0;
    HBM_TRY(hipMemGetInfo(&free_b, &total_b));
    const size_t margin = size_t(6) << 30;                              // left to everybody else while sorting
    if (free_b < margin + (3 * need + PROBES) * chunk) return hipErrorOutOfMemory;
    size_t n = (free_b - margin) / chunk;

    Sorting s;
    s.chunk = chunk;
    HBM_TRY(hipEventCreate(&s.e0));
    HBM_TRY(hipEventCreate(&s.e1));
    void *va = nullptr;
    HBM_TRY(hipMemAddressReserve(&va, n * chunk, 0, nullptr, 0));
    s.va = static_cast<char *>(va);
    s.va_bytes = n * chunk;
    hipMemAccessDesc acc = {};
    acc.location.type = hipMemLocationTypeDevice;
    acc.location.id = device;
    acc.flags = hipMemAccessFlagsProtReadWrite;
    s.handle.reserve(n); s.mapped.reserve(n); s.owned.reserve(n);
    for (size_t i = 0; i < n; ++i) {
        hipMemGenericAllocationHandle_t h;
        const hipError_t e = hipMemCreate(&h, chunk, &prop, 0);
        if (e == hipErrorOutOfMemory) { (void)hipGetLastError(); break; }   // somebody else took memory meanwhile
        HBM_TRY(e);
        s.handle.push_back(h); s.owned.push_back(1); s.mapped.push_back(0);
        HBM_TRY(hipMemMap(s.at(i), chunk, 0, h, 0));
        s.mapped[i] = 1;
        HBM_TRY(hipMemSetAccess(s.at(i), chunk, &acc, 1));
    }
    n = s.handle.size();
    if (n < 3 * need + PROBES) return hipErrorOutOfMemory;

    // 1. which kinds are there?  PROBES chunks spread over the order of creation, every pair copied both ways
    size_t probe[PROBES];
    for (int p = 0; p < PROBES; ++p) probe[p] = (n * (2 * p + 1)) / (2 * PROBES);
    float pair[PROBES][PROBES] = {};
    std::vector<float> all;
    for (int a = 0; a < PROBES; ++a)
        for (int b = 0; b < a; ++b) {
            float ab = 0.f, ba = 0.f;
            HBM_TRY(s.rate(s.at(probe[b]), s.at(probe[a]), chunk, 3, &ab));
            HBM_TRY(s.rate(s.at(probe[a]), s.at(probe[b]), chunk, 3, &ba));
            pair[a][b] = pair[b][a] = 0.5f * (ab + ba);
            all.push_back(pair[a][b]);
        }
    const float threshold = two_group_threshold(all);
    // Groups of probes: every probe starts as a group of its own, and the two groups with the slowest mean copy
    // rate between them are joined until three are left (single pairs scatter by a few percent around the two
    // typical rates; means over all pairs of two groups do not).  Whether the three are real is checked below.
    int kind[PROBES];
    for (int a = 0; a < PROBES; ++a) kind[a] = a;
    for (int groups = PROBES; groups > REGIONS; --groups) {
        int best_a = -1, best_b = -1;
        float best = 1e30f;
        for (int ga = 0; ga < PROBES; ++ga)
            for (int gb = 0; gb < ga; ++gb) {
                double sum = 0;
                int cnt = 0;
                for (int a = 0; a < PROBES; ++a)
                    for (int b = 0; b < PROBES; ++b)
                        if (kind[a] == ga && kind[b] == gb) { sum += pair[a][b]; ++cnt; }
                if (cnt && sum / cnt < best) { best = static_cast<float>(sum / cnt); best_a = ga; best_b = gb; }
            }
        for (int a = 0; a < PROBES; ++a)
            if (kind[a] == best_a) kind[a] = best_b;
    }
    // number the groups by their first probe: on a machine that has run little, region 0 is where the first
    // ordinary allocations of a process lie
    {
        int label[PROBES], next = 0;
        for (int a = 0; a < PROBES; ++a) label[a] = -1;
        for (int a = 0; a < PROBES; ++a) {
            if (label[kind[a]] < 0) label[kind[a]] = next++;
        }
        for (int a = 0; a < PROBES; ++a) kind[a] = label[kind[a]];
    }
    // real groups: between every two of them copies are clearly faster than inside either
    int kinds = REGIONS;
    for (int ga = 0; ga < REGIONS; ++ga)
        for (int gb = 0; gb < ga; ++gb) {
            double in_sum = 0, out_sum = 0;
            int in_n = 0, out_n = 0;
            for (int a = 0; a < PROBES; ++a)
                for (int b = 0; b < a; ++b) {
                    const bool a_in = kind[a] == ga || kind[a] == gb, b_in = kind[b] == ga || kind[b] == gb;
                    if (!a_in || !b_in) continue;
                    if (kind[a] == kind[b]) { in_sum += pair[a][b]; ++in_n; } else { out_sum += pair[a][b]; ++out_n; }
                }
            // (a group of one probe has no pair inside; the other group's pairs stand for both)
            if (in_n == 0 || out_n == 0 || out_sum / out_n < 1.025 * (in_sum / in_n)) kinds = REGIONS - 1;
        }
    for (int a = 0; a < PROBES; ++a) {
        rep->probe_chunk[a] = static_cast<int32_t>(probe[a]);
        rep->probe_kind[a] = kind[a];
        for (int b = 0; b < PROBES; ++b) rep->probe_pair_GBs[a][b] = pair[a][b];
    }
    rep->chunk_bytes = chunk;
    rep->chunks_examined = static_cast<int32_t>(n);
    rep->threshold_GBs = threshold;
    rep->kinds_found = kinds;
    if (kinds != REGIONS) return EXODUS_ERROR_REGIONS_NOT_FOUND;
    // the gap between the two groups of rates has to be a real one
    float slow_max = 0.f, fast_min = 1e30f, slow_sum = 0.f, fast_sum = 0.f;
    int slow_n = 0, fast_n = 0;
    for (int a = 0; a < PROBES; ++a)
        for (int b = 0; b < a; ++b) {
            if (kind[a] == kind[b]) { slow_max = std::max(slow_max, pair[a][b]); slow_sum += pair[a][b]; ++slow_n; }
            else { fast_min = std::min(fast_min, pair[a][b]); fast_sum += pair[a][b]; ++fast_n; }
        }
    if (slow_n == 0 || fast_n == 0) return EXODUS_ERROR_REGIONS_NOT_FOUND;
    rep->probe_same_kind_GBs = slow_sum / slow_n;
    rep->probe_other_kind_GBs = fast_sum / fast_n;
    if (rep->probe_other_kind_GBs < 1.025f * rep->probe_same_kind_GBs) return EXODUS_ERROR_REGIONS_NOT_FOUND;

    // 2. every chunk against up to three probes of each kind: the kind it copies to slowest
    constexpr int REFS = 3;
    int refs[REGIONS][REFS];
    for (int k = 0; k < REGIONS; ++k) {
        int cnt = 0;
        for (int r = 0; r < REFS; ++r) refs[k][r] = -1;
        for (int a = 0; a < PROBES && cnt < REFS; ++a)
            if (kind[a] == k) refs[k][cnt++] = a;
    }
    std::vector<int> kind_of(n, -1);
    for (int a = 0; a < PROBES; ++a) kind_of[probe[a]] = kind[a];
    int ambiguous = 0;
    size_t have[REGIONS] = {0, 0, 0};
    for (int a = 0; a < PROBES; ++a) ++have[kind[a]];
    for (size_t i = 0; i < n; ++i) {
        if (kind_of[i] >= 0) continue;
        if (have[0] >= need && have[1] >= need && have[2] >= need) break;   // enough of every kind
        float mean[REGIONS];
        for (int k = 0; k < REGIONS; ++k) {
            float sum = 0.f;
            int cnt = 0;
            for (int r = 0; r < REFS; ++r)
                if (refs[k][r] >= 0) {
                    float v = 0.f;
                    HBM_TRY(s.rate(s.at(probe[refs[k][r]]), s.at(i), chunk, 2, &v));
                    sum += v; ++cnt;
                }
            mean[k] = sum / cnt;
        }
        int lo = 0;
        for (int k = 1; k < REGIONS; ++k) if (mean[k] < mean[lo]) lo = k;
        float second = 1e30f;
        for (int k = 0; k < REGIONS; ++k) if (k != lo) second = std::min(second, mean[k]);
        if (mean[lo] < 0.975f * second) { kind_of[i] = lo; ++have[lo]; }
        else ++ambiguous;                                               // a chunk that spans kinds: not used
    }
    rep->chunks_ambiguous = ambiguous;
    for (int k = 0; k < REGIONS; ++k) rep->chunks_of_region[k] = static_cast<int32_t>(have[k]);
    if (have[0] < need || have[1] < need || have[2] < need) return hipErrorOutOfMemory;

    // 3. the arenas: the first `need` chunks of each kind, behind each other in a range of their own.
    // Kinds are numbered by the position of their first chunk, so that a process that comes first on a
    // machine finds region 0 where its ordinary allocations lie.
    Arenas built;
    built.chunk = chunk;
    HBM_TRY(hipDeviceSynchronize());
    int status = hipSuccess;
    for (int k = 0; k < REGIONS && status == hipSuccess; ++k) {
        void *base = nullptr;
        if ((status = hipMemAddressReserve(&base, need * chunk, 0, nullptr, 0)) != hipSuccess) break;
        built.base[k] = base;
        built.reserved[k] = need * chunk;
        for (size_t i = 0; i < n && built.handles[k].size() < need && status == hipSuccess; ++i) {
            if (kind_of[i] != k) continue;
            if ((status = hipMemUnmap(s.at(i), chunk)) != hipSuccess) break;
            s.mapped[i] = 0;
            char *dst = static_cast<char *>(base) + built.handles[k].size() * chunk;
            if ((status = hipMemMap(dst, chunk, 0, s.handle[i], 0)) != hipSuccess) break;
            s.owned[i] = 0;                                             // the arena owns the chunk from here on
            built.handles[k].push_back(s.handle[i]);
            status = hipMemSetAccess(dst, chunk, &acc, 1);
        }
    }
    auto undo = [&built]() {
        for (int k = 0; k < REGIONS; ++k) {
            for (size_t j = 0; j < built.handles[k].size(); ++j) {
                (void)hipMemUnmap(static_cast<char *>(built.base[k]) + j * built.chunk, built.chunk);
                (void)hipMemRelease(built.handles[k][j]);
            }
            if (built.base[k]) (void)hipMemAddressFree(built.base[k], built.reserved[k]);
        }
    };
    if (status != hipSuccess) { undo(); return status; }

    // 4. the proof: copies inside each arena (first half to second half) and between the arenas
    const size_t half = (need / 2) * chunk;                  // 0 when a range is one chunk
    for (int k = 0; k < REGIONS && status == hipSuccess; ++k) {
        rep->base[k] = built.base[k];
        rep->bytes[k] = need * chunk;
        rep->copy_inside_GBs[k] = 0.f;
        if (half)
            status = s.rate(static_cast<char *>(built.base[k]) + (need - need / 2) * chunk, built.base[k], half, 3,
                            &rep->copy_inside_GBs[k]);
    }
    int slot = 0;
    const size_t across = need * chunk;
    for (int j = 0; j < REGIONS && status == hipSuccess; ++j)
        for (int k = 0; k < REGIONS && status == hipSuccess; ++k)
            if (j != k) status = s.rate(built.base[k], built.base[j], across, 3, &rep->copy_across_GBs[slot++]);
    if (status != hipSuccess) { (void)hipDeviceSynchronize(); undo(); return status; }
    built.live = true;
    table[device] = std::move(built);
    return hipSuccess;          // ~Sorting returns the unused chunks
}

}  // namespace

extern "C" {

EXODUS_API int exodus_hbm_regions_create(int device, uint64_t bytes_per_region, uint64_t chunk_bytes,
                                         exodus_hbm_report *report)
{
    if (device < 0 || device >= MAX_DEVICES || !report || bytes_per_region == 0 || chunk_bytes == 0)
        return hipErrorInvalidValue;
    std::lock_guard<std::mutex> guard(table_mutex);
    if (table[device].live) return hipErrorInvalidValue;
    int before = 0;
    if (hipGetDevice(&before) != hipSuccess) return hipErrorInvalidDevice;
    *report = exodus_hbm_report{};
    const int status = create(device, bytes_per_region, chunk_bytes, report);
    (void)hipSetDevice(before);
    return status;
}

EXODUS_API int exodus_hbm_regions_destroy(int device)
{
    if (device < 0 || device >= MAX_DEVICES) return hipErrorInvalidValue;
    std::lock_guard<std::mutex> guard(table_mutex);
    Arenas &a = table[device];
    if (!a.live) return hipSuccess;
    int before = 0;
    if (hipGetDevice(&before) != hipSuccess) return hipErrorInvalidDevice;
    int status = hipSetDevice(device);
    if (status == hipSuccess) status = hipDeviceSynchronize();
    for (int k = 0; k < REGIONS; ++k) {
        for (size_t j = 0; j < a.handles[k].size(); ++j) {
            const hipError_t u = hipMemUnmap(static_cast<char *>(a.base[k]) + j * a.chunk, a.chunk);
            const hipError_t r = hipMemRelease(a.handles[k][j]);
            if (status == hipSuccess) status = u != hipSuccess ? u : r;
        }
        if (a.base[k]) {
            const hipError_t f = hipMemAddressFree(a.base[k], a.reserved[k]);
            if (status == hipSuccess) status = f;
        }
    }
    a = Arenas{};
    (void)hipSetDevice(before);
    return status;
}

}  // extern "C"
