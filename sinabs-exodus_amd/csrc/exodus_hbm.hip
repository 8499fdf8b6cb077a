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
// What costs most is writing: a kernel whose output lies in one region is held back by that region
// alone (the time-strided layer kernels write at 5.6 TB/s into one region; the (rows, time) kernels,
// which write single 128-byte lines, at 4.4-4.9), while the same kernel writing into memory whose pages
// alternate between the regions reaches 6.0-6.3 and 5.6-5.8 TB/s.  A fourth arena is therefore made of
// 64 MiB pages taken from the three regions in turn ("striped"): any tensor of a few hundred MiB in it
// spreads over all of them.  Stripes of 32 to 128 MiB measured alike; 8 MiB and 512 MiB measured worse.
// A mapping cannot start inside an allocation, so the pages have to be allocations of their own, and
// pages allocated one after the other are neighbours in physical memory only on a machine whose memory
// has never been handed out in pages before.  The pages of a known region are therefore made from a
// sorted chunk: with all other free memory held, the chunk is released and 64 pages are allocated at
// once, which can only come from the hole it left.
//
//   exodus_hbm_regions_create(device, bytes_per_region, bytes_striped, chunk_bytes, sort, take_limit_bytes, &report)
//   exodus_hbm_regions_destroy(device)
//   exodus_hbm_alloc_striped / _region0 / _region1 / _region2 (size, device, stream), exodus_hbm_free(ptr, size, device, stream)
//
// create and destroy synchronise the device.  One set of arenas per device; creating a second one fails with
// hipErrorInvalidValue until the first is destroyed.  The alloc / free pair hands out pieces of the arenas (first
// fit, pieces of 2 MiB, neighbours joined on release) in the signature of PyTorch's pluggable allocator, so that a
// torch.cuda.MemPool can sit on top: PyTorch's caching allocator then keeps track of which stream still uses
// what, and these functions only ever see whole segments come and go.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>
#include <chrono>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "exodus_common.hpp"
#include "exodus_hip.h"

#define EXODUS_API __attribute__((visibility("default")))

namespace {

constexpr int REGIONS = EXODUS_HBM_REGIONS;
constexpr int ARENAS = EXODUS_HBM_ARENAS;   // one per region and the striped one
constexpr int STRIPED = REGIONS;
constexpr size_t PAGE = EXODUS_HBM_PAGE_BYTES;
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

constexpr size_t GRANULE = size_t(2) << 20;   // pieces handed out by exodus_hbm_alloc_* are multiples of this

struct Arenas {
    bool live = false;
    void *base[ARENAS] = {nullptr, nullptr, nullptr, nullptr};
    size_t reserved[ARENAS] = {0, 0, 0, 0};
    size_t unit[ARENAS] = {0, 0, 0, 0};     // bytes per allocation: a chunk in the regions' arenas, a page in the striped one
    std::vector<hipMemGenericAllocationHandle_t> handles[ARENAS];   // allocation j is mapped at base + j * unit
    // what exodus_hbm_alloc_* has not handed out: offset -> bytes, neighbours joined; and what it has
    std::map<size_t, size_t> free_pieces[ARENAS];
    size_t in_use[ARENAS] = {0, 0, 0, 0};
    size_t pieces_out[ARENAS] = {0, 0, 0, 0};

    bool anything_out() const
    {
        for (int k = 0; k < ARENAS; ++k)
            if (pieces_out[k]) return true;
        return false;
    }

    // first fit from the lowest address; nullptr when no piece of the range is large enough
    void *take(int k, size_t bytes)
    {
        const size_t want = (bytes + GRANULE - 1) / GRANULE * GRANULE;
        for (auto it = free_pieces[k].begin(); it != free_pieces[k].end(); ++it) {
            if (it->second < want) continue;
            const size_t off = it->first, rest = it->second - want;
            free_pieces[k].erase(it);
            if (rest) free_pieces[k].emplace(off + want, rest);
            in_use[k] += want;
            ++pieces_out[k];
            return static_cast<char *>(base[k]) + off;
        }
        return nullptr;
    }

    // index of the range that holds p, or -1
    int range_of(const void *p) const
    {
        for (int k = 0; k < ARENAS; ++k)
            if (base[k] && p >= base[k] && p < static_cast<const char *>(base[k]) + reserved[k]) return k;
        return -1;
    }

    void give_back(int k, void *p, size_t bytes)
    {
        const size_t want = (bytes + GRANULE - 1) / GRANULE * GRANULE;
        size_t off = static_cast<size_t>(static_cast<char *>(p) - static_cast<char *>(base[k])), n = want;
        auto next = free_pieces[k].lower_bound(off);
        if (next != free_pieces[k].end() && off + n == next->first) {
            n += next->second;
            next = free_pieces[k].erase(next);
        }
        if (next != free_pieces[k].begin()) {
            auto prev = std::prev(next);
            if (prev->first + prev->second == off) {
                off = prev->first;
                n += prev->second;
                free_pieces[k].erase(prev);
            }
        }
        free_pieces[k].emplace(off, n);
        in_use[k] -= want;
        --pieces_out[k];
    }

    // unmaps and releases everything; returns the first error
    hipError_t release()
    {
        hipError_t status = hipSuccess;
        for (int k = 0; k < ARENAS; ++k) {
            for (size_t j = 0; j < handles[k].size(); ++j) {
                const hipError_t u = hipMemUnmap(static_cast<char *>(base[k]) + j * unit[k], unit[k]);
                const hipError_t r = hipMemRelease(handles[k][j]);
                if (status == hipSuccess) status = u != hipSuccess ? u : r;
            }
            if (base[k]) {
                const hipError_t f = hipMemAddressFree(base[k], reserved[k]);
                if (status == hipSuccess) status = f;
            }
        }
        *this = Arenas{};
        return status;
    }
};

// allocations that belong to nobody yet: released when the scope ends, unless moved on
struct Loose {
    std::vector<hipMemGenericAllocationHandle_t> handles;
    ~Loose()
    {
        for (hipMemGenericAllocationHandle_t h : handles) (void)hipMemRelease(h);
    }
};

std::mutex table_mutex;
Arenas table[MAX_DEVICES];
// what exodus_hbm_alloc_* took from the ordinary allocator because a range was absent or full: pointer -> bytes
std::unordered_map<void *, size_t> elsewhere;
size_t elsewhere_bytes[MAX_DEVICES] = {};

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

int create(int device, uint64_t bytes_per_region, uint64_t bytes_striped, uint64_t chunk_bytes, bool sort,
           uint64_t take_limit, exodus_hbm_report *rep)
{
    HBM_TRY(hipSetDevice(device));
    HBM_TRY(hipDeviceSynchronize());
    hipMemAllocationProp prop = {};
    prop.type = hipMemAllocationTypePinned;
    prop.location.type = hipMemLocationTypeDevice;
    prop.location.id = device;
    size_t gran = 0;
    HBM_TRY(hipMemGetAllocationGranularity(&gran, &prop, hipMemAllocationGranularityRecommended));
    if (gran == 0 || PAGE % gran != 0 || chunk_bytes % PAGE != 0 || chunk_bytes % (16 * 256 * COPY_PER_THREAD) != 0)
        return hipErrorInvalidValue;
    const size_t chunk = chunk_bytes;
    const size_t ppc = chunk / PAGE;                                    // pages per chunk
    const size_t need_pure = (bytes_per_region + chunk - 1) / chunk;    // chunks of each region for its own arena
    const size_t need_striped = (bytes_striped + REGIONS * chunk - 1) / (REGIONS * chunk);   // ... for the striped one
    const size_t need = need_pure + need_striped;                       // chunks wanted of each region
    size_t free_b = 0, total_b = 0;
    HBM_TRY(hipMemGetInfo(&free_b, &total_b));
    const size_t margin = size_t(6) << 30;                              // left to everybody else while sorting
    if (free_b < margin + (3 * need + PROBES) * chunk) return hipErrorOutOfMemory;
    size_t n = (free_b - margin) / chunk;
    // a caller's bound on what may be held while the ranges are made (0 = none): the part of the memory that is
    // never taken cannot be sorted, nor kept from supplying pages, so a bound trades placement for politeness
    if (take_limit) n = std::min<size_t>(n, take_limit / chunk);

    const auto clock0 = std::chrono::steady_clock::now();
    auto since = [](std::chrono::steady_clock::time_point t) {
        return std::chrono::duration<float>(std::chrono::steady_clock::now() - t).count();
    };
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
        if (!sort) continue;                       // only the timed copies need to reach the chunk's memory
        HBM_TRY(hipMemMap(s.at(i), chunk, 0, h, 0));
        s.mapped[i] = 1;
        HBM_TRY(hipMemSetAccess(s.at(i), chunk, &acc, 1));
    }
    rep->phase_s[0] = since(clock0);
    n = s.handle.size();
    if (n < 3 * need + PROBES) return hipErrorOutOfMemory;

    // 1. which kinds are there?  PROBES chunks spread over the order of creation, every pair copied both ways
    size_t probe[PROBES];
    for (int p = 0; p < PROBES; ++p) probe[p] = (n * (2 * p + 1)) / (2 * PROBES);
    float pair[PROBES][PROBES] = {};
    std::vector<float> all;
    for (int a = 0; a < PROBES && sort; ++a)
        for (int b = 0; b < a; ++b) {
            float ab = 0.f, ba = 0.f;
            HBM_TRY(s.rate(s.at(probe[b]), s.at(probe[a]), chunk, 3, &ab));
            HBM_TRY(s.rate(s.at(probe[a]), s.at(probe[b]), chunk, 3, &ba));
            pair[a][b] = pair[b][a] = 0.5f * (ab + ba);
            all.push_back(pair[a][b]);
        }
    if (!sort) all.assign(1, 0.f);                           // nothing was timed: every probe one group, no kinds
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
    // Without three kinds there are no regions to sort by: then the memory the driver hands out is already a
    // mixture at a scale below the chunks (after processes that allocated and freed it in small pieces), which
    // is what the striped range wants to be; ranges of one region cannot be made.
    bool sorted = sort && kinds == REGIONS;
    // the gap between the two groups of rates has to be a real one
    float slow_max = 0.f, fast_min = 1e30f, slow_sum = 0.f, fast_sum = 0.f;
    int slow_n = 0, fast_n = 0;
    for (int a = 0; a < PROBES; ++a)
        for (int b = 0; b < a; ++b) {
            if (kind[a] == kind[b]) { slow_max = std::max(slow_max, pair[a][b]); slow_sum += pair[a][b]; ++slow_n; }
            else { fast_min = std::min(fast_min, pair[a][b]); fast_sum += pair[a][b]; ++fast_n; }
        }
    if (slow_n == 0 || fast_n == 0) sorted = false;
    else {
        rep->probe_same_kind_GBs = slow_sum / slow_n;
        rep->probe_other_kind_GBs = fast_sum / fast_n;
        if (rep->probe_other_kind_GBs < 1.025f * rep->probe_same_kind_GBs) sorted = false;
    }
    if (!sorted) rep->kinds_found = sort ? std::min(rep->kinds_found, REGIONS - 1) : 0;
    if (!sorted && need_pure) return EXODUS_ERROR_REGIONS_NOT_FOUND;

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
    for (size_t i = 0; i < n && sorted; ++i) {
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
    if (sorted && (have[0] < need || have[1] < need || have[2] < need)) return hipErrorOutOfMemory;

    // 3. the arenas.  Of the chunks of each kind, in the order of creation, the first need_pure go behind each other
    // into the kind's own range and the next need_striped are turned into pages for the striped range.
    // Kinds are numbered by the position of their first chunk, so that a process that comes first on a
    // machine finds region 0 where its ordinary allocations lie.
    Arenas built;
    HBM_TRY(hipDeviceSynchronize());
    rep->phase_s[1] = since(clock0) - rep->phase_s[0];
    const auto clock2 = std::chrono::steady_clock::now();
    int status = hipSuccess;
    std::vector<size_t> to_pages[REGIONS];                              // chunks that become pages, by kind
    for (int k = 0; k < REGIONS && status == hipSuccess && sorted; ++k) {
        void *base = nullptr;
        if (need_pure) {
            if ((status = hipMemAddressReserve(&base, need_pure * chunk, 0, nullptr, 0)) != hipSuccess) break;
            built.base[k] = base;
            built.reserved[k] = need_pure * chunk;
            built.unit[k] = chunk;
        }
        size_t taken = 0;
        for (size_t i = 0; i < n && taken < need && status == hipSuccess; ++i) {
            if (kind_of[i] != k) continue;
            if (taken++ >= need_pure) { to_pages[k].push_back(i); continue; }
            if ((status = hipMemUnmap(s.at(i), chunk)) != hipSuccess) break;
            s.mapped[i] = 0;
            char *dst = static_cast<char *>(base) + built.handles[k].size() * chunk;
            if ((status = hipMemMap(dst, chunk, 0, s.handle[i], 0)) != hipSuccess) break;
            s.owned[i] = 0;                                             // the arena owns the chunk from here on
            built.handles[k].push_back(s.handle[i]);
            status = hipMemSetAccess(dst, chunk, &acc, 1);
        }
    }
    if (status == hipSuccess && need_striped) {
        // Pages of a known region: hold what is still free (all but half a GiB), then release one sorted chunk at
        // a time and allocate its size in pages at once -- they can only come from the hole the chunk left (a few
        // may come from the half GiB, which the striping does not notice).
        Loose held;
        size_t free_now = 0, total_now = 0;
        status = hipMemGetInfo(&free_now, &total_now);
        const size_t spare = size_t(512) << 20;
        // (with a bound on what may be taken nothing more is held: the pages then come from wherever the driver
        // finds room, which on a machine that hands memory out in address order is the hole all the same)
        while (status == hipSuccess && !take_limit && free_now > spare + PAGE) {
            hipMemGenericAllocationHandle_t h;
            const hipError_t e = hipMemCreate(&h, PAGE, &prop, 0);
            if (e == hipErrorOutOfMemory) { (void)hipGetLastError(); break; }
            if ((status = e) != hipSuccess) break;
            held.handles.push_back(h);
            free_now -= PAGE;
        }
        // the chunks whose pages take turns in the range: one of each kind after the other -- or, with no kinds,
        // chunks spread evenly over the order of creation, taken from its first, second and last third in turn
        // (on a machine that hands memory out in address order the thirds are the regions; on one that does not,
        // any order is as good)
        const size_t lanes = REGIONS * need_striped;
        std::vector<size_t> turn;
        for (size_t c = 0; c < lanes; ++c) {
            const size_t spread = (c % REGIONS) * need_striped + c / REGIONS;    // position among `lanes` even steps
            turn.push_back(sorted ? to_pages[c % REGIONS][c / REGIONS] : (n * (2 * spread + 1)) / (2 * lanes));
        }
        std::vector<Loose> pages(lanes);
        for (size_t c = 0; c < lanes && status == hipSuccess; ++c) {
            const size_t i = turn[c];
            if (s.mapped[i] && (status = hipMemUnmap(s.at(i), chunk)) != hipSuccess) break;
            s.mapped[i] = 0;
            if ((status = hipMemRelease(s.handle[i])) != hipSuccess) break;
            s.owned[i] = 0;
            for (size_t j = 0; j < ppc && status == hipSuccess; ++j) {
                hipMemGenericAllocationHandle_t h;
                if ((status = hipMemCreate(&h, PAGE, &prop, 0)) == hipSuccess) pages[c].handles.push_back(h);
            }
        }
        const size_t total = lanes * ppc;                               // pages of the striped range
        void *base = nullptr;
        if (status == hipSuccess && (status = hipMemAddressReserve(&base, total * PAGE, 0, nullptr, 0)) == hipSuccess) {
            built.base[STRIPED] = base;
            built.reserved[STRIPED] = total * PAGE;
            built.unit[STRIPED] = PAGE;
            // page q of the range is page q / lanes of chunk q mod lanes; the arena owns a page once it is mapped
            for (size_t q = 0; q < total && status == hipSuccess; ++q) {
                const hipMemGenericAllocationHandle_t h = pages[q % lanes].handles[q / lanes];
                if ((status = hipMemMap(static_cast<char *>(base) + q * PAGE, PAGE, 0, h, 0)) != hipSuccess) break;
                built.handles[STRIPED].push_back(h);
            }
            // the pages that were mapped are the first ones of each chunk's list, in turn
            for (size_t c = 0; c < lanes; ++c) {
                const size_t mapped_c = (built.handles[STRIPED].size() + lanes - 1 - c) / lanes;
                pages[c].handles.erase(pages[c].handles.begin(), pages[c].handles.begin() + mapped_c);
            }
            if (status == hipSuccess) status = hipMemSetAccess(base, total * PAGE, &acc, 1);
        }
    }                                                                   // what was held goes back here
    if (status != hipSuccess) { (void)built.release(); return status; }

    rep->phase_s[2] = since(clock2);
    const auto clock3 = std::chrono::steady_clock::now();
    // 4. the proof: copies inside each arena (first half to second half) and between the regions' arenas
    const size_t half = (need_pure / 2) * chunk;             // 0 when a range is one chunk or absent
    for (int k = 0; k < ARENAS; ++k) {
        rep->base[k] = built.base[k];
        rep->bytes[k] = built.reserved[k];
    }
    rep->page_bytes = PAGE;
    for (int k = 0; k < REGIONS && status == hipSuccess; ++k) {
        rep->copy_inside_GBs[k] = 0.f;
        if (half)
            status = s.rate(static_cast<char *>(built.base[k]) + (need_pure - need_pure / 2) * chunk, built.base[k], half, 3,
                            &rep->copy_inside_GBs[k]);
    }
    int slot = 0;
    const size_t across = need_pure * chunk;
    for (int j = 0; j < REGIONS && status == hipSuccess && across; ++j)
        for (int k = 0; k < REGIONS && status == hipSuccess; ++k)
            if (j != k) status = s.rate(built.base[k], built.base[j], across, 3, &rep->copy_across_GBs[slot++]);
    rep->copy_striped_GBs = 0.f;
    if (status == hipSuccess && need_striped) {
        const size_t h = built.reserved[STRIPED] / (2 * chunk) * chunk;
        if (h) status = s.rate(static_cast<char *>(built.base[STRIPED]) + h, built.base[STRIPED], h, 3, &rep->copy_striped_GBs);
    }
    if (status != hipSuccess) { (void)hipDeviceSynchronize(); (void)built.release(); return status; }
    rep->phase_s[3] = since(clock3);
    for (int k = 0; k < ARENAS; ++k)
        if (built.reserved[k]) built.free_pieces[k].emplace(size_t(0), built.reserved[k]);
    built.live = true;
    table[device] = std::move(built);
    return hipSuccess;          // ~Sorting returns the unused chunks
}

}  // namespace

extern "C" {

EXODUS_API int exodus_hbm_regions_create(int device, uint64_t bytes_per_region, uint64_t bytes_striped,
                                         uint64_t chunk_bytes, int sort, uint64_t take_limit_bytes,
                                         exodus_hbm_report *report)
{
    if (device < 0 || device >= MAX_DEVICES || !report || (bytes_per_region == 0 && bytes_striped == 0) || chunk_bytes == 0)
        return hipErrorInvalidValue;
    if (!sort && bytes_per_region != 0) return hipErrorInvalidValue;    // ranges of one region need the sorting
    std::lock_guard<std::mutex> guard(table_mutex);
    if (table[device].live) return hipErrorInvalidValue;
    int before = 0;
    if (hipGetDevice(&before) != hipSuccess) return hipErrorInvalidDevice;
    *report = exodus_hbm_report{};
    const int status = create(device, bytes_per_region, bytes_striped, chunk_bytes, sort != 0, take_limit_bytes, report);
    (void)hipSetDevice(before);
    return status;
}

EXODUS_API int exodus_hbm_regions_destroy(int device)
{
    if (device < 0 || device >= MAX_DEVICES) return hipErrorInvalidValue;
    std::lock_guard<std::mutex> guard(table_mutex);
    Arenas &a = table[device];
    if (!a.live) return hipSuccess;
    if (a.anything_out()) return EXODUS_ERROR_RANGE_IN_USE;     // memory that somebody still holds is never unmapped
    int before = 0;
    if (hipGetDevice(&before) != hipSuccess) return hipErrorInvalidDevice;
    int status = hipSetDevice(device);
    if (status == hipSuccess) status = hipDeviceSynchronize();
    const hipError_t released = a.release();
    if (status == hipSuccess) status = released;
    (void)hipSetDevice(before);
    return status;
}

// A piece of range `k` of `device`, or -- when the device has no such range, or the range no room -- plain device
// memory (remembered, so that exodus_hbm_free knows what to do with it): a caller of these functions is an
// allocator that cannot do anything useful with a null pointer.
static void *alloc_from(int k, size_t size, int device)
{
    if (device < 0 || device >= MAX_DEVICES) return nullptr;
    if (size == 0) size = 1;
    std::lock_guard<std::mutex> guard(table_mutex);
    Arenas &a = table[device];
    if (a.live && a.base[k]) {
        if (void *p = a.take(k, size)) return p;
    }
    int before = 0;
    if (hipGetDevice(&before) != hipSuccess) return nullptr;
    void *p = nullptr;
    if (hipSetDevice(device) == hipSuccess && hipMalloc(&p, size) != hipSuccess) {
        (void)hipGetLastError();
        p = nullptr;
    }
    (void)hipSetDevice(before);
    if (p) {
        elsewhere[p] = size;
        elsewhere_bytes[device] += size;
    }
    return p;
}

EXODUS_API void *exodus_hbm_alloc_striped(size_t size, int device, void *) { return alloc_from(STRIPED, size, device); }
EXODUS_API void *exodus_hbm_alloc_region0(size_t size, int device, void *) { return alloc_from(0, size, device); }
EXODUS_API void *exodus_hbm_alloc_region1(size_t size, int device, void *) { return alloc_from(1, size, device); }
EXODUS_API void *exodus_hbm_alloc_region2(size_t size, int device, void *) { return alloc_from(2, size, device); }

EXODUS_API void exodus_hbm_free(void *ptr, size_t size, int device, void *)
{
    if (!ptr || device < 0 || device >= MAX_DEVICES) return;
    if (size == 0) size = 1;
    std::lock_guard<std::mutex> guard(table_mutex);
    Arenas &a = table[device];
    const int k = a.live ? a.range_of(ptr) : -1;
    if (k >= 0) {
        a.give_back(k, ptr, size);
        return;
    }
    auto it = elsewhere.find(ptr);
    if (it == elsewhere.end()) return;                          // not from here: nothing this library may free
    elsewhere_bytes[device] -= it->second;
    elsewhere.erase(it);
    int before = 0;
    if (hipGetDevice(&before) != hipSuccess) return;
    if (hipSetDevice(device) == hipSuccess) (void)hipFree(ptr);
    (void)hipSetDevice(before);
}

EXODUS_API int exodus_hbm_usage(int device, uint64_t *bytes_in_use, uint64_t *bytes_elsewhere)
{
    if (device < 0 || device >= MAX_DEVICES || !bytes_in_use) return hipErrorInvalidValue;
    std::lock_guard<std::mutex> guard(table_mutex);
    for (int k = 0; k < ARENAS; ++k) bytes_in_use[k] = table[device].live ? table[device].in_use[k] : 0;
    if (bytes_elsewhere) *bytes_elsewhere = elsewhere_bytes[device];
    return hipSuccess;
}

}  // extern "C"
