// libexodus_hip.so -- gfx950 kernels for the EXODUS neuron-dynamics path and their C ABI.
//
// Layout problem: tensors are (rows, steps) with time contiguous, the recurrences are
// sequential in time and independent across rows.  One lane owns one row.  A wave owns 64
// consecutive rows and walks the time axis in tiles of TT steps:
//
//   global -> registers : each row segment of TT floats is fetched by TT/4 adjacent lanes as
//                         16-byte vectors, so a wave-wide load touches whole contiguous segments
//   registers -> LDS    : stored as a [64 rows][TT] tile whose 16-byte chunks are XOR-swizzled
//   LDS -> lane         : lane r reads row r chunk by chunk (conflict free thanks to the swizzle),
//                         runs the recurrence for 4 steps per chunk and writes results in place
//   LDS -> global       : same mapping as the load, again whole segments
//
// The next tile's global loads are issued before the current tile is computed, so HBM latency
// overlaps the serial dependency chain.  Tiles are private to a wave (workgroup = one wave), so
// no workgroup barrier exists anywhere; ordering between the phases only needs the in-order
// execution of one wave's LDS instructions plus a compiler fence.
//
// Two drivers implement this scheme: scan_span_kernel for rows whose length is a multiple of 4 in
// 16-byte aligned tensors (raw buffer instructions on the wave's span of memory, sectors shared by two
// rows written whole), scan_kernel for everything else (global loads, element-wise at row boundaries).
//
// Arithmetic of the forward recurrences is written with explicit round-to-nearest multiplies and
// adds (no fused multiply-add), in the operation order of the reference device code, so spike
// trains are reproducible bit for bit against a scalar CPU evaluation.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "exodus_hip.h"
#include "exodus_common.hpp"

namespace {

template <int TT>
struct Geom {
    static_assert(TT == 16 || TT == 32 || TT == 64, "tile length");
    static constexpr int CPR = TT / 4;                       // 16-byte chunks per row segment
    static constexpr int RPI = WAVE / CPR;                   // rows fetched by one wave-wide load
    static constexpr int NLD = CPR;                          // wave-wide loads per tile (64 rows / RPI)
    static constexpr int ROWS_PER_BANK_LINE = (CPR >= 16) ? 1 : 16 / CPR;   // rows per 256 B of LDS
    // float offset of logical chunk `c` of row `r` inside a tile
    __device__ static __forceinline__ int off(int r, int c)
    {
        return r * TT + 4 * (c ^ ((r / ROWS_PER_BANK_LINE) & (CPR - 1)));
    }
};

// `keep`: an ordinary load instead of a streaming one, for lines that another tile will ask for again
template <class T> __device__ __forceinline__ T ld_pick(const T *p, bool keep)
{
    return keep ? *p : ld_stream(p);
}

__device__ __forceinline__ f32x4 load4(const float *__restrict__ base, int64_t row, int64_t n_rows,
                                       int64_t t, int64_t n_steps, bool keep)
{
    // t may be negative (before the row's first step) or beyond the row's end: those lanes load nothing
    f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
    if (row < n_rows) {
        const float *p = base + row * n_steps + t;
        if (t >= 0 && t + 3 < n_steps && (reinterpret_cast<uintptr_t>(p) & 15u) == 0) {
            // rows of any length: tiles are aligned to memory, so a chunk that lies inside its row is a
            // 16-byte aligned vector; only the chunks that straddle a row boundary go element by element
            v = ld_pick(reinterpret_cast<const f32x4 *>(p), keep);
        } else {
            if (t + 0 >= 0 && t + 0 < n_steps) v.x = ld_pick(p + 0, keep);
            if (t + 1 >= 0 && t + 1 < n_steps) v.y = ld_pick(p + 1, keep);
            if (t + 2 >= 0 && t + 2 < n_steps) v.z = ld_pick(p + 2, keep);
            if (t + 3 >= 0 && t + 3 < n_steps) v.w = ld_pick(p + 3, keep);
        }
    }
    return v;
}

__device__ __forceinline__ void store4(float *__restrict__ base, int64_t row, int64_t n_rows, int64_t t,
                                       int64_t n_steps, f32x4 v)
{
    if (row < n_rows) {
        float *p = base + row * n_steps + t;
        if (t >= 0 && t + 3 < n_steps && (reinterpret_cast<uintptr_t>(p) & 15u) == 0) {
            st_stream(v, reinterpret_cast<f32x4 *>(p));
        } else {
            if (t + 0 >= 0 && t + 0 < n_steps) st_stream(v.x, p + 0);
            if (t + 1 >= 0 && t + 1 < n_steps) st_stream(v.y, p + 1);
            if (t + 2 >= 0 && t + 2 < n_steps) st_stream(v.z, p + 2);
            if (t + 3 >= 0 && t + 3 < n_steps) st_stream(v.w, p + 3);
        }
    }
}

__device__ __forceinline__ float get(const f32x4 &v, int e) { return v[e]; }
__device__ __forceinline__ void put(f32x4 &v, int e, float x) { v[e] = x; }

// ---------------------------------------------------------------------------------------------
// The scan driver.  Op supplies:
//   NIN, NOUT          number of (n,t) inputs / outputs; output j reuses the LDS slot of input j
//   REVERSE            walk time from the last step to the first
//   in[NIN], out[NOUT] device pointers
//   State, init(State&, row, valid), step(State&, const float* x, float* y), end_tile(State&)
//   (called after each tile), finish(State&, row)
//   NDER (0 or 1)      one more (n,t) output that is a pure function of output DER_SRC and of
//                      NROWP per-row constants: it is computed while the tile is written back
//                      (stash(State&, float* p) / derive(const float* p, f32x4 v)), so it needs no
//                      LDS tile of its own
//
// Tiles are aligned to memory, not to the rows.  Row r starts at float offset base + r*n_steps,
// which in general is not a multiple of the tile length, so a tile that started at the row's first
// step would straddle 128-byte lines on every access.  Instead tile k of row r covers the steps
// [k*TT - shift_r, (k+1)*TT - shift_r) with shift_r = (base + r*n_steps) mod TT: every wave-wide
// load and store then moves whole aligned TT*4-byte segments, and only the first and last tile
// of a row are partial (their out-of-row steps are masked per lane).
// ---------------------------------------------------------------------------------------------
template <class Op, int TT>
__global__ void __launch_bounds__(WAVE) scan_kernel(const Op op, const int64_t n_rows, const int64_t n_steps,
                                                    const int64_t n_tiles, const int base_shift)
{
    using G = Geom<TT>;
    constexpr int NIN = Op::NIN, NOUT = Op::NOUT;
    constexpr int NSLOT = NIN > NOUT ? NIN : NOUT;
    constexpr int TILE = WAVE * TT;                           // floats per tile
    constexpr int NDER = Op::NDER, NROWP = Op::NROWP;
    extern __shared__ f32x4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    float *rowp = lds + NSLOT * TILE;                         // [64 rows][NROWP] constants for derive()

    const int lane = threadIdx.x;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * WAVE;
    const int64_t my_row = row0 + lane;
    const bool row_ok = my_row < n_rows;

    typename Op::State st;
    op.init(st, row_ok ? my_row : n_rows - 1, row_ok);
    if constexpr (NDER > 0) {
        float consts[NROWP > 0 ? NROWP : 1];
        op.stash(st, consts);
#pragma unroll
        for (int k = 0; k < NROWP; ++k) rowp[lane * NROWP + k] = consts[k];
    }

    const int l_chunk = lane % G::CPR;                        // which 16 B of the segment this lane moves
    const int l_row = lane / G::CPR;                          // first row this lane moves
    // misalignment of a row's first step relative to a TT-float boundary
    auto shift_of = [&](int64_t row) { return static_cast<int>((base_shift + row * n_steps) & (TT - 1)); };
    const int my_shift = shift_of(my_row);
    int mv_shift[G::NLD];                                     // shifts of the rows this lane moves
#pragma unroll
    for (int i = 0; i < G::NLD; ++i) mv_shift[i] = shift_of(row0 + l_row + i * G::RPI);

    f32x4 pre[NIN > 0 ? NIN : 1][G::NLD];

    // a row's first and last tile hold the lines it shares with the neighbouring rows, which fetch them
    // many tiles away in time: those loads are left cacheable, all others stream (stores always stream:
    // cacheable stores to the shared lines measured 15 % slower on short rows)
    auto edge_tile = [&](int64_t tile) { return !(tile >= 1 && (tile + 1) * TT <= n_steps); };
    auto fetch = [&](int64_t tile) {
        const bool keep = edge_tile(tile);
#pragma unroll
        for (int i = 0; i < G::NLD; ++i) {
            const int64_t t = tile * TT - mv_shift[i] + 4 * l_chunk;
#pragma unroll
            for (int j = 0; j < NIN; ++j)
                pre[j][i] = load4(op.in[j], row0 + l_row + i * G::RPI, n_rows, t, n_steps, keep);
        }
    };

    // the recurrence over one tile: lane = row, 4 steps per 16-byte chunk.  GUARD masks the steps
    // that fall outside the row (first and last tile only).
    auto compute = [&](int64_t t_first, auto guard) {
        constexpr bool GUARD = decltype(guard)::value;
        EXODUS_UNROLL(EXODUS_UNROLL_Q)
        for (int qq = 0; qq < G::CPR; ++qq) {
            const int q = Op::REVERSE ? G::CPR - 1 - qq : qq;
            f32x4 xin[NIN > 0 ? NIN : 1];
            f32x4 yout[NOUT > 0 ? NOUT : 1];
#pragma unroll
            for (int j = 0; j < NIN; ++j)
                xin[j] = *reinterpret_cast<const f32x4 *>(lds + j * TILE + G::off(lane, q));
#pragma unroll
            for (int j = 0; j < NOUT; ++j) yout[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ee = 0; ee < 4; ++ee) {
                const int e = Op::REVERSE ? 3 - ee : ee;
                const int64_t t = t_first + 4 * q + e;
                if (!GUARD || (t >= 0 && t < n_steps)) {
                    float x[NIN > 0 ? NIN : 1];
                    float y[NOUT > 0 ? NOUT : 1];
#pragma unroll
                    for (int j = 0; j < NIN; ++j) x[j] = get(xin[j], e);
                    op.step(st, x, y);
#pragma unroll
                    for (int j = 0; j < NOUT; ++j) put(yout[j], e, y[j]);
                }
            }
#pragma unroll
            for (int j = 0; j < NOUT; ++j)
                *reinterpret_cast<f32x4 *>(lds + j * TILE + G::off(lane, q)) = yout[j];
        }
    };

    fetch(Op::REVERSE ? n_tiles - 1 : 0);

    for (int64_t it = 0; it < n_tiles; ++it) {
        const int64_t tile = Op::REVERSE ? n_tiles - 1 - it : it;

        // registers -> LDS
#pragma unroll
        for (int j = 0; j < NIN; ++j)
#pragma unroll
            for (int i = 0; i < G::NLD; ++i)
                *reinterpret_cast<f32x4 *>(lds + j * TILE + G::off(l_row + i * G::RPI, l_chunk)) = pre[j][i];

        // next tile's loads stay in flight during the compute and store phases below
        if (it + 1 < n_tiles) fetch(Op::REVERSE ? tile - 1 : tile + 1);

        wave_sync();

        // a tile is interior when it lies inside the row for every possible shift (0..TT-1)
        const bool interior = tile >= 1 && (tile + 1) * TT <= n_steps;
        if (interior)
            compute(tile * TT - my_shift, std::false_type{});
        else
            compute(tile * TT - my_shift, std::true_type{});
        op.end_tile(st);

        if (NOUT > 0) {
            wave_sync();
            // LDS -> global, whole aligned segments per group of CPR lanes
#pragma unroll
            for (int i = 0; i < G::NLD; ++i) {
                const int64_t t = tile * TT - mv_shift[i] + 4 * l_chunk;
#pragma unroll
                for (int j = 0; j < NOUT; ++j) {
                    const f32x4 v = *reinterpret_cast<const f32x4 *>(lds + j * TILE + G::off(l_row + i * G::RPI, l_chunk));
                    store4(op.out[j], row0 + l_row + i * G::RPI, n_rows, t, n_steps, v);
                    if constexpr (NDER > 0) {
                        if (j == Op::DER_SRC)
                            store4(op.der, row0 + l_row + i * G::RPI, n_rows, t, n_steps,
                                        op.derive(rowp + (l_row + i * G::RPI) * NROWP, v));
                    }
                }
            }
        }
        wave_sync();
    }

    if (row_ok) op.finish(st, my_row);
}

// ---------------------------------------------------------------------------------------------
// The same driver for the common case (row length a multiple of 4, 16-byte aligned tensors), with raw
// buffer instructions.  A wave's 64 rows are one contiguous span of memory, at most 2^30 bytes long, so
// every access is  span base (resource descriptor in SGPRs) + 32-bit lane offset:
//   * no 64-bit address arithmetic and no per-access bounds code: one offset register per wave-wide
//     load (shared by all tensors) plus the tile's offset; the driver above spends 170-370 registers
//     on addresses, hoisted tile reads and prefetch data and keeps 1-3 waves per SIMD resident, this
//     one 4-6, which is what hides the chains of dependent instructions of the recurrences;
//   * the descriptor's size ends the span at the last valid row, so rows past the end of the tensor
//     read zeros and drop their stores in hardware;
//   * a row's first and last tiles share their memory lines with the neighbouring rows: there a lane
//     whose 16 bytes lie outside its row gets an offset beyond the span (reads zero, stores nothing).
// UQ = chunks of 4 steps the recurrence loop is unrolled by (caps how many tile reads are hoisted).
// ---------------------------------------------------------------------------------------------
typedef __amdgpu_buffer_rsrc_t Rsrc;
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
constexpr unsigned OUTSIDE = 0x80000000u;                     // an offset beyond any span

__device__ __forceinline__ Rsrc span_rsrc(const float *base, unsigned bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(base), 0, static_cast<int>(bytes), 0x00020000);
}
template <bool STREAM> __device__ __forceinline__ f32x4 span_load(Rsrc r, unsigned off)
{
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, (STREAM && EXODUS_NT_LOAD) ? 2 : 0));
}
__device__ __forceinline__ void span_store(f32x4 v, Rsrc r, unsigned off)
{
    // the whole offset travels in the vector register and a short wait that reads the data follows: a 16-byte
    // buffer store with a scalar offset, directly followed by a write to its data registers, has stored wrong
    // values on gfx950
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), r, off, 0, EXODUS_NT_STORE ? 2 : 0);
    asm volatile("s_nop 1" : : "v"(v));
}

template <class Op, int TT, int UQ, int WPE>
__global__ void __launch_bounds__(WAVE) __attribute__((amdgpu_waves_per_eu(WPE, WPE)))
scan_span_kernel(const Op op, const int64_t n_rows, const int n_steps, const int n_tiles, const int base_shift,
                 const int whole_sectors)
{
    using G = Geom<TT>;
    constexpr int NIN = Op::NIN, NOUT = Op::NOUT;
    constexpr int NSLOT = NIN > NOUT ? NIN : NOUT;
    constexpr int TILE = WAVE * TT;
    constexpr int NDER = Op::NDER, NROWP = Op::NROWP;
    extern __shared__ f32x4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    float *rowp = lds + NSLOT * TILE;
    float *kept_back = rowp + WAVE * NROWP;                   // [NOUT][64 rows][4 chunks] with whole_sectors

    const int lane = threadIdx.x;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * WAVE;
    const int n_loc = n_rows - row0 < WAVE ? static_cast<int>(n_rows - row0) : WAVE;   // rows of this wave
    const bool row_ok = lane < n_loc;

    typename Op::State st;
    op.init(st, row_ok ? row0 + lane : n_rows - 1, row_ok);
    if constexpr (NDER > 0) {
        float consts[NROWP > 0 ? NROWP : 1];
        op.stash(st, consts);
#pragma unroll
        for (int k = 0; k < NROWP; ++k) rowp[lane * NROWP + k] = consts[k];
    }

    // the span: from the tile boundary at or below the first row's first step to the last row's end
    const int64_t e0 = row0 * n_steps;
    const int d = static_cast<int>((base_shift + e0) & (TT - 1));
    const unsigned span_bytes = 4u * static_cast<unsigned>(d + n_loc * n_steps);
    Rsrc rin[NIN > 0 ? NIN : 1], rout[NOUT > 0 ? NOUT : 1], rder;
#pragma unroll
    for (int j = 0; j < NIN; ++j) rin[j] = span_rsrc(op.in[j] + (e0 - d), span_bytes);
#pragma unroll
    for (int j = 0; j < NOUT; ++j) rout[j] = span_rsrc(op.out[j] + (e0 - d), span_bytes);
    if constexpr (NDER > 0) rder = span_rsrc(op.der + (e0 - d), span_bytes);

    const int l_chunk = lane % G::CPR;
    const int l_row = lane / G::CPR;
    // float position of a row's first step inside the span, and its distance from the tile boundary below
    auto start_of = [&](int r) { return d + r * n_steps; };
    const int my_shift = start_of(lane) & (TT - 1);
    unsigned voff[G::NLD];                                    // byte offset of this lane's 16 bytes in tile 0
#pragma unroll
    for (int i = 0; i < G::NLD; ++i)
        voff[i] = 4u * static_cast<unsigned>(start_of(l_row + i * G::RPI) & ~(TT - 1)) + 16u * l_chunk;
    // first and last tiles: the offset, or OUTSIDE where the 16 bytes are not part of the row
    auto edge_off = [&](int tile, int i) {
        const int r = l_row + i * G::RPI;
        const int t = tile * TT - (start_of(r) & (TT - 1)) + 4 * l_chunk;
        return (r < n_loc && t >= 0 && t + 3 < n_steps) ? voff[i] + static_cast<unsigned>(tile) * (TT * 4u) : OUTSIDE;
    };
    auto interior = [&](int tile) { return tile >= 1 && (tile + 1) * TT <= n_steps; };

    f32x4 pre[NIN > 0 ? NIN : 1][G::NLD];
    auto fetch = [&](int tile) {
        if (interior(tile)) {
            const unsigned toff = static_cast<unsigned>(tile) * (TT * 4u);
#pragma unroll
            for (int i = 0; i < G::NLD; ++i)
#pragma unroll
                for (int j = 0; j < NIN; ++j) pre[j][i] = span_load<true>(rin[j], voff[i] + toff);
        } else {
            // lines shared with the neighbouring rows, which ask for them many tiles away in time: cacheable
#pragma unroll
            for (int i = 0; i < G::NLD; ++i) {
                const unsigned off = edge_off(tile, i);
#pragma unroll
                for (int j = 0; j < NIN; ++j) pre[j][i] = span_load<false>(rin[j], off);
            }
        }
    };

    auto compute = [&](int t_first, auto guard) {
        constexpr bool GUARD = decltype(guard)::value;
        EXODUS_UNROLL(UQ)
        for (int qq = 0; qq < G::CPR; ++qq) {
            const int q = Op::REVERSE ? G::CPR - 1 - qq : qq;
            f32x4 xin[NIN > 0 ? NIN : 1];
            f32x4 yout[NOUT > 0 ? NOUT : 1];
#pragma unroll
            for (int j = 0; j < NIN; ++j)
                xin[j] = *reinterpret_cast<const f32x4 *>(lds + j * TILE + G::off(lane, q));
#pragma unroll
            for (int j = 0; j < NOUT; ++j) yout[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ee = 0; ee < 4; ++ee) {
                const int e = Op::REVERSE ? 3 - ee : ee;
                const int t = t_first + 4 * q + e;
                if (!GUARD || static_cast<unsigned>(t) < static_cast<unsigned>(n_steps)) {
                    float x[NIN > 0 ? NIN : 1];
                    float y[NOUT > 0 ? NOUT : 1];
#pragma unroll
                    for (int j = 0; j < NIN; ++j) x[j] = get(xin[j], e);
                    op.step(st, x, y);
#pragma unroll
                    for (int j = 0; j < NOUT; ++j) put(yout[j], e, y[j]);
                }
            }
#pragma unroll
            for (int j = 0; j < NOUT; ++j)
                *reinterpret_cast<f32x4 *>(lds + j * TILE + G::off(lane, q)) = yout[j];
        }
    };

    fetch(Op::REVERSE ? n_tiles - 1 : 0);

    for (int it = 0; it < n_tiles; ++it) {
        const int tile = Op::REVERSE ? n_tiles - 1 - it : it;
#pragma unroll
        for (int j = 0; j < NIN; ++j)
#pragma unroll
            for (int i = 0; i < G::NLD; ++i)
                *reinterpret_cast<f32x4 *>(lds + j * TILE + G::off(l_row + i * G::RPI, l_chunk)) = pre[j][i];

        if (it + 1 < n_tiles) fetch(Op::REVERSE ? tile - 1 : tile + 1);

        wave_sync();
        const bool inner = interior(tile);
        if (inner)
            compute(tile * TT - my_shift, std::false_type{});
        else
            compute(tile * TT - my_shift, std::true_type{});
        op.end_tile(st);

        if (NOUT > 0 && inner) {
            wave_sync();
#pragma unroll
            for (int i = 0; i < G::NLD; ++i) {
                const unsigned off = voff[i] + static_cast<unsigned>(tile) * (TT * 4u);
#pragma unroll
                for (int j = 0; j < NOUT; ++j) {
                    const f32x4 v = *reinterpret_cast<const f32x4 *>(lds + j * TILE + G::off(l_row + i * G::RPI, l_chunk));
                    span_store(v, rout[j], off);
                    if constexpr (NDER > 0) {
                        if (j == Op::DER_SRC)
                            span_store(op.derive(rowp + (l_row + i * G::RPI) * NROWP, v), rder, off);
                    }
                }
            }
        } else if (NOUT > 0) {
            // A row's first and last tile.  Where rows do not start on 64-byte boundaries, the sector that holds the
            // end of one row and the start of the next would be written in two parts, many tiles apart in time (a
            // partial write costs the memory a read and a write).  With whole_sectors the part that is produced first
            // -- the next row's first values when time runs forward, the row's last values when it runs backward --
            // is kept back in LDS and leaves together with the other part, through the lanes that hold that part's
            // line anyway.  Only the sectors between the rows of two waves stay split.
            wave_sync();
#pragma unroll
            for (int i = 0; i < G::NLD; ++i) {
                const int r = l_row + i * G::RPI;
                const int sh = start_of(r) & (TT - 1);
                const int t = tile * TT - sh + 4 * l_chunk;
                const bool in_row = r < n_loc && t >= 0 && t + 3 < n_steps;
                unsigned off = in_row ? voff[i] + static_cast<unsigned>(tile) * (TT * 4u) : OUTSIDE;
                bool keep = false, kept = false;              // this lane's values stay here / come from what was kept
                int src = r;                                  // the row whose values this lane stores
                if (whole_sectors) {
                    const int sector = tile * (TT / 16) + (l_chunk >> 2);   // of this lane's 16 bytes, from the row's tile 0
                    const int e = sh + n_steps;                             // where the next row starts, likewise
                    if (!Op::REVERSE) {
                        keep = in_row && r >= 1 && (sh & 15) != 0 && sector == (sh >> 4);
                        kept = !in_row && r + 1 < n_loc && t >= n_steps && (e & 15) != 0 && sector == (e >> 4);
                        if (kept) src = r + 1;
                    } else {
                        keep = in_row && r + 1 < n_loc && (e & 15) != 0 && sector == (e >> 4);
                        kept = !in_row && r >= 1 && r < n_loc && t < 0 && (sh & 15) != 0 && sector == (sh >> 4);
                        if (kept) src = r - 1;
                    }
                    if (kept) off = voff[i] + static_cast<unsigned>(tile) * (TT * 4u);
                    if (keep) off = OUTSIDE;
                }
#pragma unroll
                for (int j = 0; j < NOUT; ++j) {
                    f32x4 v = *reinterpret_cast<const f32x4 *>(lds + j * TILE + G::off(r, l_chunk));
                    f32x4 *slot = reinterpret_cast<f32x4 *>(kept_back + ((j * WAVE + src) * 4 + (l_chunk & 3)) * 4);
                    if (keep) *slot = v;
                    if (kept) v = *slot;
                    span_store(v, rout[j], off);
                    if constexpr (NDER > 0) {
                        if (j == Op::DER_SRC) span_store(op.derive(rowp + src * NROWP, v), rder, off);
                    }
                }
            }
        }
        wave_sync();
    }

    if (row_ok) op.finish(st, row0 + lane);
}

// ---------------------------------------------------------------------------------------------
// Ops
// ---------------------------------------------------------------------------------------------
struct LeakyFwdOp {
    static constexpr int NDER = 0, NROWP = 0;
    static constexpr int NIN = 1, NOUT = 1;
    static constexpr bool REVERSE = false;
    const float *in[1];
    float *out[1];
    const float *v_init, *alpha;
    struct State { float v, a; };
    __device__ __forceinline__ void init(State &s, int64_t row, bool) const
    {
        s.v = v_init[row];
        s.a = alpha[row];
    }
    __device__ __forceinline__ void step(State &s, const float *x, float *y) const
    {
        s.v = __fadd_rn(__fmul_rn(s.v, s.a), x[0]);
        y[0] = s.v;
    }
    __device__ __forceinline__ void end_tile(State &) const {}
    __device__ __forceinline__ void finish(State &, int64_t) const {}
};

// reverse pass of the leaky integrator; optional alpha gradient and optional input-gradient store
template <bool ALPHA, bool WRITE_GI>
struct LeakyBwdOp {
    static constexpr int NDER = 0, NROWP = 0;
    static constexpr int NIN = ALPHA ? 2 : 1, NOUT = WRITE_GI ? 1 : 0;
    static constexpr bool REVERSE = true;
    const float *in[NIN];                                     // [0] output_grad, [1] forward output
    float *out[1];
    const float *v_init, *alpha;
    float *alpha_grad, *init_grad;
    struct State { float g, a; TileSum acc; };
    __device__ __forceinline__ void init(State &s, int64_t row, bool) const
    {
        s.g = 0.f;
        s.a = alpha[row];
        s.acc.clear();
    }
    __device__ __forceinline__ void step(State &s, const float *x, float *y) const
    {
        if (ALPHA) s.acc.add(s.g, x[1]);                          // g_{u+1} * out_u
        s.g = __fadd_rn(__fmul_rn(s.g, s.a), x[0]);
        if (WRITE_GI) y[0] = s.g;
    }
    __device__ __forceinline__ void end_tile(State &s) const { if (ALPHA) s.acc.fold(); }
    __device__ __forceinline__ void finish(State &s, int64_t row) const
    {
        if (init_grad) init_grad[row] = __fmul_rn(s.a, s.g);
        if (ALPHA) {
            s.acc.add(s.g, v_init[row]);
            s.acc.fold();
            alpha_grad[row] = static_cast<float>(s.acc.total);
        }
    }
};

__device__ __forceinline__ f32x4 spike_count4(f32x4 v, float theta, unsigned cap)
{
    return f32x4{spike_count(v.x, theta, cap), spike_count(v.y, theta, cap), spike_count(v.z, theta, cap),
                 spike_count(v.w, theta, cap)};
}

struct LifFwdOp {
    // out[0] = v_mem (in place of x); the spike raster is a function of v_mem and the row's
    // threshold, so it is produced on the way out instead of occupying a second tile
    static constexpr int NIN = 1, NOUT = 1, NDER = 1, NROWP = 1, DER_SRC = 0;
    static constexpr bool REVERSE = false;
    const float *in[1];
    float *out[1];
    float *der;
    const float *v_init, *alpha, *c, *theta, *theta_low;
    int apply_low;
    unsigned cap;
    struct State { float v, a, c, th, lo, cnt; };
    __device__ __forceinline__ void init(State &s, int64_t row, bool) const
    {
        s.v = v_init[row];
        s.a = alpha[row];
        s.c = c[row];
        s.th = theta[row];
        s.lo = apply_low ? theta_low[row] : 0.f;
        s.cnt = 0.f;
    }
    __device__ __forceinline__ void stash(const State &s, float *p) const { p[0] = s.th; }
    __device__ __forceinline__ f32x4 derive(const float *p, f32x4 v) const { return spike_count4(v, p[0], cap); }
    __device__ __forceinline__ void step(State &s, const float *x, float *y) const
    {
        float v = __fsub_rn(s.v, __fmul_rn(s.cnt, s.c));
        v = __fmul_rn(v, s.a);
        v = __fadd_rn(v, x[0]);
        if (apply_low && v < s.lo) v = s.lo;
        s.cnt = spike_count(v, s.th, cap);
        s.v = v;
        y[0] = v;
    }
    __device__ __forceinline__ void end_tile(State &) const {}
    __device__ __forceinline__ void finish(State &, int64_t) const {}
};

// Synapse + membrane in one pass (what the layer otherwise composes from a scaling, a leaky
// integrator, another scaling and the spiking stage):
//   xin = decay_early ? x * a_syn : x;   i = i * a_syn + xin;   u = norm_input ? (1 - a_mem) * i : i
//   v = (v - count*c) * a_mem + u;  clamp;  count from v
// out[0] = v_mem (in place of x), out[1] = i_syn, derived = spikes
struct SynLifFwdOp {
    static constexpr int NIN = 1, NOUT = 2, NDER = 1, NROWP = 1, DER_SRC = 0;
    static constexpr bool REVERSE = false;
    const float *in[1];
    float *out[2];
    float *der;
    const float *v_init, *i_init, *alpha_mem, *alpha_syn, *c, *theta, *theta_low;
    int apply_low, decay_early, norm_input;
    unsigned cap;
    struct State { float v, i, am, as, k, c, th, lo, cnt; };
    __device__ __forceinline__ void init(State &s, int64_t row, bool) const
    {
        s.v = v_init[row];
        s.i = i_init[row];
        s.am = alpha_mem[row];
        s.as = alpha_syn[row];
        s.k = __fsub_rn(1.0f, s.am);
        s.c = c[row];
        s.th = theta[row];
        s.lo = apply_low ? theta_low[row] : 0.f;
        s.cnt = 0.f;
    }
    __device__ __forceinline__ void stash(const State &s, float *p) const { p[0] = s.th; }
    __device__ __forceinline__ f32x4 derive(const float *p, f32x4 v) const { return spike_count4(v, p[0], cap); }
    __device__ __forceinline__ void step(State &s, const float *x, float *y) const
    {
        const float xin = decay_early ? __fmul_rn(x[0], s.as) : x[0];
        s.i = __fadd_rn(__fmul_rn(s.i, s.as), xin);
        const float u = norm_input ? __fmul_rn(s.k, s.i) : s.i;
        float v = __fsub_rn(s.v, __fmul_rn(s.cnt, s.c));
        v = __fmul_rn(v, s.am);
        v = __fadd_rn(v, u);
        if (apply_low && v < s.lo) v = s.lo;
        s.cnt = spike_count(v, s.th, cap);
        s.v = v;
        y[0] = v;
        y[1] = s.i;
    }
    __device__ __forceinline__ void end_tile(State &) const {}
    __device__ __forceinline__ void finish(State &, int64_t) const {}
};

// One reverse pass for the spiking layer: input gradient, initial-state gradient and alpha gradient.
//   slot 0: grad wrt spikes (in) / input gradient (out);  slot 1: v_mem;  then grad wrt v_mem
//   (HAS_GV) and the surrogate tensor (KIND == EXODUS_SURR_TENSOR)
template <int KIND, bool HAS_GV, bool ALPHA>
struct LifBwdOp {
    static constexpr int NDER = 0, NROWP = 0;
    static constexpr int GV_SLOT = 2, SURR_SLOT = HAS_GV ? 3 : 2;
    static constexpr int NIN = 2 + (HAS_GV ? 1 : 0) + (KIND == EXODUS_SURR_TENSOR ? 1 : 0), NOUT = 1;
    static constexpr bool REVERSE = true;
    const float *in[NIN];
    float *out[1];
    const float *v_init, *alpha, *c, *theta, *theta_low;
    float *alpha_grad, *init_grad;
    int apply_low;
    unsigned cap;
    float p0, p1, inv_p0;
    struct State { float lam, a, ac, c, th, lo; SurrConst k; TileSum acc; };
    __device__ __forceinline__ void init(State &s, int64_t row, bool) const
    {
        s.lam = 0.f;
        s.a = alpha[row];
        s.c = c[row];
        s.ac = __fmul_rn(s.a, s.c);
        s.th = theta[row];
        s.lo = apply_low ? theta_low[row] : 0.f;
        s.acc.clear();
        if constexpr (KIND != EXODUS_SURR_TENSOR) s.k = surrogate_consts<KIND>(s.th, p0, p1);
    }
    __device__ __forceinline__ void step(State &s, const float *x, float *y) const
    {
        const float v = x[1];
        float sg;
        if constexpr (KIND == EXODUS_SURR_TENSOR) sg = x[SURR_SLOT];
        else sg = surrogate<KIND>(v, s.th, inv_p0, s.k);
        float g = __fmul_rn(sg, x[0]);
        if constexpr (HAS_GV) g = __fadd_rn(g, x[GV_SLOT]);
        if (ALPHA) {
            const float vpost = __fsub_rn(v, __fmul_rn(s.c, spike_count(v, s.th, cap)));
            s.acc.add(s.lam, vpost);                              // lambda_{u+1} * vpost_u
        }
        const float f = __fsub_rn(s.a, __fmul_rn(s.ac, sg));
        const float lam = __fadd_rn(g, __fmul_rn(f, s.lam));
        s.lam = (apply_low && !(v > s.lo)) ? 0.f : lam;
        y[0] = s.lam;
    }
    __device__ __forceinline__ void end_tile(State &s) const { if (ALPHA) s.acc.fold(); }
    __device__ __forceinline__ void finish(State &s, int64_t row) const
    {
        if (init_grad) init_grad[row] = __fmul_rn(s.a, s.lam);
        if (ALPHA) {
            s.acc.add(s.lam, v_init[row]);
            s.acc.fold();
            alpha_grad[row] = static_cast<float>(s.acc.total);
        }
    }
};

// Reverse pass of the fused synapse + membrane stage.  With lambda_t = dL/du_t (membrane adjoint)
// and mu_t = dL/di_t (synapse adjoint):
//   lambda_t = nc_t (g_t + (a_mem - a_mem c s_t) lambda_{t+1}),   g_t = s_t * grad_spikes_t [+ grad_vmem_t]
//   mu_t     = a_syn mu_{t+1} + k lambda_t [+ grad_isyn_t],       k = norm_input ? 1 - a_mem : 1
//   grad_x_t = decay_early ? a_syn mu_t : mu_t
//   grad_alpha_mem = sum_t lambda_t vpost_{t-1}  -  (norm_input ? sum_t lambda_t i_t : 0)
//   grad_alpha_syn = decay_early ? (sum_t mu_t i_t) / a_syn : sum_t mu_t i_{t-1}
//   grad_v_init = a_mem lambda_0,  grad_i_init = a_syn mu_0
// slots: 0 grad_spikes (in) / grad_x (out), 1 v_mem, 2 i_syn, then grad_vmem and grad_isyn (EXTRA)
template <int KIND, bool EXTRA>
struct SynLifBwdOp {
    static_assert(KIND != EXODUS_SURR_TENSOR, "the fused stage evaluates its surrogate in-kernel");
    static constexpr int NDER = 0, NROWP = 0;
    static constexpr int NIN = EXTRA ? 5 : 3, NOUT = 1;
    static constexpr bool REVERSE = true;
    const float *in[NIN];
    float *out[1];
    const float *v_init, *i_init, *alpha_mem, *alpha_syn, *c, *theta, *theta_low;
    float *alpha_mem_grad, *alpha_syn_grad, *v_init_grad, *i_init_grad;
    int apply_low, decay_early, norm_input;
    unsigned cap;
    float p0, p1, inv_p0;
    struct State { float lam, mu, am, as, amc, k, c, th, lo; SurrConst sk; TileSum acc_m, acc_s; };
    __device__ __forceinline__ void init(State &s, int64_t row, bool) const
    {
        s.lam = 0.f;
        s.mu = 0.f;
        s.am = alpha_mem[row];
        s.as = alpha_syn[row];
        s.c = c[row];
        s.amc = __fmul_rn(s.am, s.c);
        s.k = norm_input ? __fsub_rn(1.0f, s.am) : 1.0f;
        s.th = theta[row];
        s.lo = apply_low ? theta_low[row] : 0.f;
        s.acc_m.clear();
        s.acc_s.clear();
        s.sk = surrogate_consts<KIND>(s.th, p0, p1);
    }
    __device__ __forceinline__ void step(State &s, const float *x, float *y) const
    {
        const float v = x[1], i = x[2];
        const float sg = surrogate<KIND>(v, s.th, inv_p0, s.sk);
        float g = __fmul_rn(sg, x[0]);
        if constexpr (EXTRA) g = __fadd_rn(g, x[3]);
        const float vpost = __fsub_rn(v, __fmul_rn(s.c, spike_count(v, s.th, cap)));
        s.acc_m.add(s.lam, vpost);                                // lambda_{u+1} * vpost_u
        if (!decay_early) s.acc_s.add(s.mu, i);                   // mu_{u+1} * i_u
        const float f = __fsub_rn(s.am, __fmul_rn(s.amc, sg));
        const float lam = __fadd_rn(g, __fmul_rn(f, s.lam));
        s.lam = (apply_low && !(v > s.lo)) ? 0.f : lam;
        if (norm_input) s.acc_m.sub(s.lam, i);
        float du = __fmul_rn(s.lam, s.k);
        if constexpr (EXTRA) du = __fadd_rn(du, x[4]);
        s.mu = __fadd_rn(__fmul_rn(s.mu, s.as), du);
        if (decay_early) s.acc_s.add(s.mu, i);                    // mu_u * i_u
        y[0] = decay_early ? __fmul_rn(s.mu, s.as) : s.mu;
    }
    __device__ __forceinline__ void end_tile(State &s) const
    {
        s.acc_m.fold();
        s.acc_s.fold();
    }
    __device__ __forceinline__ void finish(State &s, int64_t row) const
    {
        if (v_init_grad) v_init_grad[row] = __fmul_rn(s.am, s.lam);
        if (i_init_grad) i_init_grad[row] = __fmul_rn(s.as, s.mu);
        if (alpha_mem_grad) {
            s.acc_m.add(s.lam, v_init[row]);
            s.acc_m.fold();
            alpha_mem_grad[row] = static_cast<float>(s.acc_m.total);
        }
        if (alpha_syn_grad) {
            if (decay_early) {
                s.acc_s.total = s.acc_s.total / static_cast<double>(s.as);
            } else {
                s.acc_s.add(s.mu, i_init[row]);
                s.acc_s.fold();
            }
            alpha_syn_grad[row] = static_cast<float>(s.acc_s.total);
        }
    }
};

// counterpart of the reference's lifBackward: surrogate, g and the clip mask come as tensors
struct LifBwdTensorsOp {
    static constexpr int NDER = 0, NROWP = 0;
    static constexpr int NIN = 3, NOUT = 1;                   // in: g, surr, not_clipped
    static constexpr bool REVERSE = true;
    const float *in[3];
    float *out[1];
    const float *alpha, *csub;
    struct State { float lam, a, cs; };
    __device__ __forceinline__ void init(State &s, int64_t row, bool) const
    {
        s.lam = 0.f;
        s.a = alpha[row];
        s.cs = csub[row];
    }
    __device__ __forceinline__ void step(State &s, const float *x, float *y) const
    {
        const float f = __fsub_rn(s.a, __fmul_rn(s.cs, x[1]));
        s.lam = __fmul_rn(x[2], __fadd_rn(x[0], __fmul_rn(f, s.lam)));
        y[0] = s.lam;
    }
    __device__ __forceinline__ void end_tile(State &) const {}
    __device__ __forceinline__ void finish(State &, int64_t) const {}
};

// counterpart of the reference's lifBackwardAlpha: forward in time, D recurrence
struct LifBwdAlphaTensorsOp {
    static constexpr int NDER = 0, NROWP = 0;
    static constexpr int NIN = 4, NOUT = 0;                   // in: g, surr, not_clipped, v_post
    static constexpr bool REVERSE = false;
    const float *in[4];
    float *out[1];
    const float *v_init, *alpha, *c;
    float *alpha_grad;
    int gate_initial;
    struct State { float d, a, c, s_prev, vp_prev; double acc; bool first; };
    __device__ __forceinline__ void init(State &s, int64_t row, bool) const
    {
        s.d = v_init[row];
        s.a = alpha[row];
        s.c = c[row];
        s.s_prev = 0.f;
        s.vp_prev = 0.f;
        s.acc = 0.0;
        s.first = true;
    }
    __device__ __forceinline__ void step(State &s, const float *x, float *) const
    {
        if (s.first) {
            const float d0 = __fmul_rn(x[2], s.d);
            s.acc = static_cast<double>(d0) * static_cast<double>(x[0]);
            if (gate_initial) s.d = d0;
            s.first = false;
        } else {
            // D = D * (alpha * (1 - c*s_prev)) with the factor formed in double, as the reference's
            // "1.0 -" literal makes it
            const double fac = static_cast<double>(s.a) * (1.0 - static_cast<double>(__fmul_rn(s.c, s.s_prev)));
            float d = static_cast<float>(static_cast<double>(s.d) * fac);
            d = __fadd_rn(d, s.vp_prev);
            d = __fmul_rn(d, x[2]);
            s.d = d;
            s.acc += static_cast<double>(d) * static_cast<double>(x[0]);
        }
        s.s_prev = x[1];
        s.vp_prev = x[3];
    }
    __device__ __forceinline__ void end_tile(State &) const {}
    __device__ __forceinline__ void finish(State &s, int64_t row) const { alpha_grad[row] = static_cast<float>(s.acc); }
};

// Spike generation on a membrane potential that already holds the response to the input (the
// reference's experimental spikeForward): only reset and lower bound act.  The reference subtracts
// alpha^j * c * count from every later step for each spike, one spike after the other; here the sum
// of all pending corrections is one running value  adj_t = alpha * (adj_{t-1} + d_{t-1})  with
// d = -c * count after a spike and d = theta_low - u below the lower bound, which is the same
// real-number result in O(T) instead of O(T^2) (float rounding differs in the last bits).
// out[0] = corrected potential, written over the input; spikes are derived from it on the way out.
struct SpikeFwdOp {
    static constexpr int NIN = 1, NOUT = 1, NDER = 1, NROWP = 1, DER_SRC = 0;
    static constexpr bool REVERSE = false;
    const float *in[1];
    float *out[1];
    float *der;
    float alpha, c, theta, theta_low;
    int apply_low;
    unsigned cap;
    struct State { float adj; };
    __device__ __forceinline__ void init(State &s, int64_t, bool) const { s.adj = 0.f; }
    __device__ __forceinline__ void stash(const State &, float *p) const { p[0] = theta; }
    __device__ __forceinline__ f32x4 derive(const float *p, f32x4 v) const { return spike_count4(v, p[0], cap); }
    __device__ __forceinline__ void step(State &s, const float *x, float *y) const
    {
        const float u = __fadd_rn(x[0], s.adj);
        y[0] = u;
        float d = 0.f;
        if (u >= theta)
            d = -__fmul_rn(c, spike_count(u, theta, cap));
        else if (apply_low && u < theta_low)
            d = __fsub_rn(theta_low, u);
        s.adj = __fmul_rn(alpha, __fadd_rn(s.adj, d));
    }
    __device__ __forceinline__ void end_tile(State &) const {}
    __device__ __forceinline__ void finish(State &, int64_t) const {}
};

// Its backward (the reference's experimental spikeBackward), with y = surr * not_clipped:
//   gi_i = y_i go_i - (y_i c) m_i,   m_i = go_{i+1} y_{i+1} + (alpha - c y_{i+1}) m_{i+1},  m_{T-1} = 0
// which is the reference's per-element sum over j > i written as one reverse pass.
struct SpikeBwdOp {
    static constexpr int NDER = 0, NROWP = 0;
    static constexpr int NIN = 3, NOUT = 1;                   // in: grad_out, surr, not_clipped
    static constexpr bool REVERSE = true;
    const float *in[3];
    float *out[1];
    float alpha, c;
    struct State { float m; };
    __device__ __forceinline__ void init(State &s, int64_t, bool) const { s.m = 0.f; }
    __device__ __forceinline__ void step(State &s, const float *x, float *y) const
    {
        const float g = __fmul_rn(x[1], x[2]);
        const float gy = __fmul_rn(g, x[0]);
        y[0] = __fsub_rn(gy, __fmul_rn(__fmul_rn(g, c), s.m));
        s.m = __fadd_rn(gy, __fmul_rn(__fsub_rn(alpha, __fmul_rn(c, g)), s.m));
    }
    __device__ __forceinline__ void end_tile(State &) const {}
    __device__ __forceinline__ void finish(State &, int64_t) const {}
};

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------

// Tile length, unrolling and register budget of the span driver by the number of tiles an op keeps in LDS.
// A wave's LDS footprint is slots * 64 rows * TT steps * 4 bytes of the CU's 160 KB; the register budget is
// set to the number of waves per SIMD that this footprint allows (at most EXODUS_WPE_MAX).
template <class Op>
struct SpanPlan {
    static constexpr int NSLOT = Op::NIN > Op::NOUT ? Op::NIN : Op::NOUT;
    static constexpr int TT = NSLOT >= 3 ? EXODUS_TT_S3 : (NSLOT == 2 ? EXODUS_TT_S2 : EXODUS_TT_S1);
    static constexpr int LDS_BYTES = (NSLOT * WAVE * TT + WAVE * Op::NROWP) * 4;
    static constexpr int PER_CU = (160 * 1024) / LDS_BYTES;
    static constexpr int WPE_LDS = (PER_CU + 3) / 4;
    static constexpr int WPE = WPE_LDS < 1 ? 1 : (WPE_LDS > EXODUS_WPE_MAX ? EXODUS_WPE_MAX : WPE_LDS);
    static constexpr int UQ = EXODUS_SPAN_UNROLL_Q;
};

template <class Op, int TT>
int launch_rows(const Op &op, int64_t n, int64_t t, bool vec, void *stream)
{
    constexpr int NSLOT = Op::NIN > Op::NOUT ? Op::NIN : Op::NOUT;
    const size_t lds_bytes = (static_cast<size_t>(NSLOT) * WAVE * TT + WAVE * Op::NROWP) * sizeof(float);
    const int64_t n_blocks = (n + WAVE - 1) / WAVE;
    if (n_blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    // Tiles are aligned to the first tensor's address (allocators hand out >= 256-byte aligned
    // blocks, so in practice every tensor shares this alignment).  Row shifts are
    // (base_shift + r*t) mod TT, i.e. base_shift plus multiples of g = gcd(t, TT); the largest one
    // decides how many tiles cover a row.
    const void *first = Op::NIN > 0 ? static_cast<const void *>(op.in[0]) : static_cast<const void *>(op.out[0]);
    const int base_shift = static_cast<int>((reinterpret_cast<uintptr_t>(first) / sizeof(float)) % TT);
    int64_t g = t % TT == 0 ? TT : t % TT;
    for (int64_t b = TT; b != 0;) { const int64_t r = g % b; g = b; b = r; }    // gcd(t mod TT, TT)
    const int64_t max_shift = TT - g + (base_shift % g);
    const int64_t n_tiles = (t - 1 + max_shift) / TT + 1;
    const dim3 grid(static_cast<unsigned>(n_blocks)), block(WAVE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if constexpr (TT == SpanPlan<Op>::TT) {
        // 64 rows of at most 2^22 steps: a wave's span stays below 2^30 bytes
        if (vec && t <= (1 << 22)) {
            // rows that do not all start on 64-byte boundaries: sectors shared by two rows are written whole, which
            // takes 4 chunks of LDS per row and output (rows of at least a tile, so that a row's two ends lie in
            // different tiles)
            const int whole_sectors = EXODUS_WHOLE_SECTORS && Op::NOUT > 0 && t > TT && (t % 16 != 0 || base_shift % 16 != 0);
            const size_t lds_kept = whole_sectors ? static_cast<size_t>(Op::NOUT) * WAVE * 16 * sizeof(float) : 0;
            hipLaunchKernelGGL((scan_span_kernel<Op, TT, SpanPlan<Op>::UQ, SpanPlan<Op>::WPE>), grid, block,
                               lds_bytes + lds_kept + EXODUS_SPAN_EXTRA_LDS, s, op, n, static_cast<int>(t), static_cast<int>(n_tiles), base_shift,
                               whole_sectors);
            return static_cast<int>(hipGetLastError());
        }
    }
    hipLaunchKernelGGL((scan_kernel<Op, TT>), grid, block, lds_bytes, s, op, n, t, n_tiles, base_shift);
    return static_cast<int>(hipGetLastError());
}

// `TT_GENERIC` is the tile length of the driver for rows of any length and alignment
template <class Op, int TT_GENERIC>
int launch(const Op &op, int64_t n, int64_t t, void *stream)
{
    bool vec = (t % 4) == 0;
    for (int j = 0; j < Op::NIN; ++j) vec = vec && aligned16(op.in[j]);
    for (int j = 0; j < Op::NOUT; ++j) vec = vec && aligned16(op.out[j]);
    if constexpr (Op::NDER > 0) vec = vec && aligned16(op.der);   // the derived output leaves through the same stores
    if (vec && t <= (1 << 22)) return launch_rows<Op, SpanPlan<Op>::TT>(op, n, t, true, stream);
    return launch_rows<Op, TT_GENERIC>(op, n, t, false, stream);
}

inline bool bad_dims(int64_t n, int64_t t) { return n < 0 || t < 0 || (t > 0 && n > INT64_MAX / t); }

template <int KIND, bool HAS_GV, bool ALPHA>
int launch_lif_bwd(float *input_grad, float *alpha_grad, float *init_grad, const float *grad_spikes,
                   const float *grad_vmem, const float *vmem, const float *surr, const float *v_init,
                   const float *alpha, const float *c, const float *theta, const float *theta_low,
                   int apply_low, int max_spikes, float p0, float p1, int64_t n, int64_t t, void *stream)
{
    using Op = LifBwdOp<KIND, HAS_GV, ALPHA>;
    Op op;
    op.in[0] = grad_spikes;
    op.in[1] = vmem;
    if constexpr (HAS_GV) op.in[Op::GV_SLOT] = grad_vmem;
    if constexpr (KIND == EXODUS_SURR_TENSOR) op.in[Op::SURR_SLOT] = surr;
    op.out[0] = input_grad;
    op.v_init = v_init;
    op.alpha = alpha;
    op.c = c;
    op.theta = theta;
    op.theta_low = theta_low;
    op.alpha_grad = alpha_grad;
    op.init_grad = init_grad;
    op.apply_low = apply_low;
    op.cap = static_cast<unsigned>(max_spikes);
    op.p0 = p0;
    op.p1 = p1;
    op.inv_p0 = p0 != 0.f ? 1.f / p0 : 0.f;
    if constexpr (Op::NIN <= 2) return launch<Op, EXODUS_TT_1>(op, n, t, stream);
    else return launch<Op, EXODUS_TT_3>(op, n, t, stream);
}

template <int KIND>
int dispatch_lif_bwd(bool has_gv, bool want_alpha, float *input_grad, float *alpha_grad, float *init_grad,
                     const float *grad_spikes, const float *grad_vmem, const float *vmem, const float *surr,
                     const float *v_init, const float *alpha, const float *c, const float *theta,
                     const float *theta_low, int apply_low, int max_spikes, float p0, float p1, int64_t n,
                     int64_t t, void *stream)
{
#define EXODUS_CALL(GV, AL)                                                                                     \
    return launch_lif_bwd<KIND, GV, AL>(input_grad, alpha_grad, init_grad, grad_spikes, grad_vmem, vmem, surr, \
                                        v_init, alpha, c, theta, theta_low, apply_low, max_spikes, p0, p1, n,  \
                                        t, stream)
    if (has_gv) {
        if (want_alpha) EXODUS_CALL(true, true);
        EXODUS_CALL(true, false);
    }
    if (want_alpha) EXODUS_CALL(false, true);
    EXODUS_CALL(false, false);
#undef EXODUS_CALL
}

template <int KIND, bool EXTRA>
int launch_synlif_bwd(float *grad_input, float *alpha_mem_grad, float *alpha_syn_grad, float *v_init_grad,
                      float *i_init_grad, const float *grad_spikes, const float *grad_vmem, const float *grad_isyn,
                      const float *vmem, const float *isyn, const float *v_init, const float *i_init,
                      const float *alpha_mem, const float *alpha_syn, const float *c, const float *theta,
                      const float *theta_low, int apply_low, int max_spikes, int decay_early, int norm_input,
                      float p0, float p1, int64_t n, int64_t t, void *stream)
{
    using Op = SynLifBwdOp<KIND, EXTRA>;
    Op op;
    op.in[0] = grad_spikes;
    op.in[1] = vmem;
    op.in[2] = isyn;
    if constexpr (EXTRA) {
        op.in[3] = grad_vmem;
        op.in[4] = grad_isyn;
    }
    op.out[0] = grad_input;
    op.v_init = v_init;
    op.i_init = i_init;
    op.alpha_mem = alpha_mem;
    op.alpha_syn = alpha_syn;
    op.c = c;
    op.theta = theta;
    op.theta_low = theta_low;
    op.alpha_mem_grad = alpha_mem_grad;
    op.alpha_syn_grad = alpha_syn_grad;
    op.v_init_grad = v_init_grad;
    op.i_init_grad = i_init_grad;
    op.apply_low = apply_low;
    op.decay_early = decay_early;
    op.norm_input = norm_input;
    op.cap = static_cast<unsigned>(max_spikes);
    op.p0 = p0;
    op.p1 = p1;
    op.inv_p0 = p0 != 0.f ? 1.f / p0 : 0.f;
    return launch<Op, EXODUS_TT_3>(op, n, t, stream);
}

}  // namespace

// ---------------------------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------------------------
extern "C" {

#define EXODUS_API __attribute__((visibility("default")))

EXODUS_API int exodus_hip_abi_version(void) { return EXODUS_HIP_ABI_VERSION; }

EXODUS_API const char *exodus_hip_error_string(int status)
{
    if (status == EXODUS_ERROR_SCRATCH_TOO_SMALL)
        return "one batch element needs more checkpoint memory than the library's fixed scratch array holds "
               "(see exodus_layer_scratch_floats); use exodus_layer_lif_forward / exodus_layer_lif_backward with "
               "caller-allocated checkpoints";
    if (status == EXODUS_ERROR_REGIONS_NOT_FOUND)
        return "timed copies between chunks of device memory did not show three kinds of chunks with a clear gap "
               "between them: this device's memory has no regions to sort tensors by, or something else was "
               "using it during the measurement";
    if (status == EXODUS_ERROR_RANGE_IN_USE)
        return "memory handed out by exodus_hbm_alloc_* has not come back through exodus_hbm_free yet: the ranges "
               "stay as they are";
    return hipGetErrorString(static_cast<hipError_t>(status));
}

EXODUS_API int exodus_lif_forward(float *out_spikes, float *out_vmem, const float *input,
                                  const float *vmem_post_initial, const float *alpha,
                                  const float *membr_subtract, const float *theta, const float *theta_low,
                                  int apply_theta_low, int max_num_spikes, int64_t n, int64_t t, void *stream)
{
    if (bad_dims(n, t)) return hipErrorInvalidValue;
    if (n == 0 || t == 0) return hipSuccess;
    if (!out_spikes || !out_vmem || !input || !vmem_post_initial || !alpha || !membr_subtract || !theta ||
        (apply_theta_low && !theta_low))
        return hipErrorInvalidValue;
    LifFwdOp op;
    op.in[0] = input;
    op.out[0] = out_vmem;
    op.der = out_spikes;
    op.v_init = vmem_post_initial;
    op.alpha = alpha;
    op.c = membr_subtract;
    op.theta = theta;
    op.theta_low = theta_low;
    op.apply_low = apply_theta_low ? 1 : 0;
    op.cap = static_cast<unsigned>(max_num_spikes);           // negative -> no cap
    return launch<LifFwdOp, EXODUS_TT_1>(op, n, t, stream);
}

EXODUS_API int exodus_lif_backward(float *input_grad, const float *surr, const float *output_grad,
                                   const float *not_clipped, const float *alpha, const float *membr_subtract,
                                   int64_t n, int64_t t, void *stream)
{
    if (bad_dims(n, t)) return hipErrorInvalidValue;
    if (n == 0 || t == 0) return hipSuccess;
    if (!input_grad || !surr || !output_grad || !not_clipped || !alpha || !membr_subtract)
        return hipErrorInvalidValue;
    LifBwdTensorsOp op;
    op.in[0] = output_grad;
    op.in[1] = surr;
    op.in[2] = not_clipped;
    op.out[0] = input_grad;
    op.alpha = alpha;
    op.csub = membr_subtract;
    return launch<LifBwdTensorsOp, EXODUS_TT_3>(op, n, t, stream);
}

EXODUS_API int exodus_lif_backward_alpha(float *alpha_grad, const float *surr, const float *output_grad,
                                         const float *vmem_post, const float *vmem_post_initial,
                                         const float *not_clipped, const float *alpha,
                                         const float *membr_subtract, int gate_initial, int64_t n, int64_t t,
                                         void *stream)
{
    if (bad_dims(n, t)) return hipErrorInvalidValue;
    if (n == 0 || t == 0) return hipSuccess;
    if (!alpha_grad || !surr || !output_grad || !vmem_post || !vmem_post_initial || !not_clipped || !alpha ||
        !membr_subtract)
        return hipErrorInvalidValue;
    LifBwdAlphaTensorsOp op;
    op.in[0] = output_grad;
    op.in[1] = surr;
    op.in[2] = not_clipped;
    op.in[3] = vmem_post;
    op.out[0] = nullptr;
    op.v_init = vmem_post_initial;
    op.alpha = alpha;
    op.c = membr_subtract;
    op.alpha_grad = alpha_grad;
    op.gate_initial = gate_initial ? 1 : 0;
    return launch<LifBwdAlphaTensorsOp, EXODUS_TT_3>(op, n, t, stream);
}

EXODUS_API int exodus_leaky_forward(float *out, const float *input, const float *vmem_initial,
                                    const float *alpha, int64_t n, int64_t t, void *stream)
{
    if (bad_dims(n, t)) return hipErrorInvalidValue;
    if (n == 0 || t == 0) return hipSuccess;
    if (!out || !input || !vmem_initial || !alpha) return hipErrorInvalidValue;
    LeakyFwdOp op;
    op.in[0] = input;
    op.out[0] = out;
    op.v_init = vmem_initial;
    op.alpha = alpha;
    return launch<LeakyFwdOp, EXODUS_TT_1>(op, n, t, stream);
}

EXODUS_API int exodus_leaky_backward_fused(float *input_grad, float *alpha_grad, float *init_grad,
                                           const float *output_grad, const float *output,
                                           const float *vmem_initial, const float *alpha, int64_t n, int64_t t,
                                           void *stream)
{
    if (bad_dims(n, t)) return hipErrorInvalidValue;
    if (n == 0 || t == 0) return hipSuccess;
    if (!output_grad || !alpha) return hipErrorInvalidValue;
    if (alpha_grad && (!output || !vmem_initial)) return hipErrorInvalidValue;
    if (!input_grad && !alpha_grad) return hipErrorInvalidValue;
    if (alpha_grad) {
        if (input_grad) {
            LeakyBwdOp<true, true> op;
            op.in[0] = output_grad; op.in[1] = output; op.out[0] = input_grad;
            op.v_init = vmem_initial; op.alpha = alpha; op.alpha_grad = alpha_grad; op.init_grad = init_grad;
            return launch<LeakyBwdOp<true, true>, EXODUS_TT_1>(op, n, t, stream);
        }
        LeakyBwdOp<true, false> op;
        op.in[0] = output_grad; op.in[1] = output; op.out[0] = nullptr;
        op.v_init = vmem_initial; op.alpha = alpha; op.alpha_grad = alpha_grad; op.init_grad = init_grad;
        return launch<LeakyBwdOp<true, false>, EXODUS_TT_1>(op, n, t, stream);
    }
    LeakyBwdOp<false, true> op;
    op.in[0] = output_grad; op.out[0] = input_grad;
    op.v_init = vmem_initial; op.alpha = alpha; op.alpha_grad = nullptr; op.init_grad = init_grad;
    return launch<LeakyBwdOp<false, true>, EXODUS_TT_1>(op, n, t, stream);
}

EXODUS_API int exodus_leaky_backward(float *input_grad, const float *output_grad, const float *alpha,
                                     int64_t n, int64_t t, void *stream)
{
    if (!input_grad) return hipErrorInvalidValue;
    return exodus_leaky_backward_fused(input_grad, nullptr, nullptr, output_grad, nullptr, nullptr, alpha, n, t,
                                       stream);
}

EXODUS_API int exodus_leaky_backward_alpha(float *alpha_grad, const float *output_grad, const float *output,
                                           const float *vmem_initial, const float *alpha, int64_t n, int64_t t,
                                           void *stream)
{
    if (!alpha_grad) return hipErrorInvalidValue;
    return exodus_leaky_backward_fused(nullptr, alpha_grad, nullptr, output_grad, output, vmem_initial, alpha, n,
                                       t, stream);
}

EXODUS_API int exodus_lif_backward_fused(float *input_grad, float *alpha_grad, float *init_grad,
                                         const float *grad_spikes, const float *grad_vmem, const float *vmem,
                                         const float *surr, const float *vmem_post_initial, const float *alpha,
                                         const float *membr_subtract, const float *theta, const float *theta_low,
                                         int apply_theta_low, int max_num_spikes, int surrogate_kind,
                                         float surr_p0, float surr_p1, int64_t n, int64_t t, void *stream)
{
    if (bad_dims(n, t)) return hipErrorInvalidValue;
    if (n == 0 || t == 0) return hipSuccess;
    if (!input_grad || !grad_spikes || !vmem || !alpha || !membr_subtract || !theta) return hipErrorInvalidValue;
    if (apply_theta_low && !theta_low) return hipErrorInvalidValue;
    if (alpha_grad && !vmem_post_initial) return hipErrorInvalidValue;
    if (surrogate_kind == EXODUS_SURR_TENSOR && !surr) return hipErrorInvalidValue;
    const bool gv = grad_vmem != nullptr, al = alpha_grad != nullptr;
#define EXODUS_KIND(K)                                                                                         \
    return dispatch_lif_bwd<K>(gv, al, input_grad, alpha_grad, init_grad, grad_spikes, grad_vmem, vmem, surr, \
                               vmem_post_initial, alpha, membr_subtract, theta, theta_low,                    \
                               apply_theta_low ? 1 : 0, max_num_spikes, surr_p0, surr_p1, n, t, stream)
    switch (surrogate_kind) {
        case EXODUS_SURR_TENSOR: EXODUS_KIND(EXODUS_SURR_TENSOR);
        case EXODUS_SURR_SINGLE_EXP: EXODUS_KIND(EXODUS_SURR_SINGLE_EXP);
        case EXODUS_SURR_PERIODIC_EXP: EXODUS_KIND(EXODUS_SURR_PERIODIC_EXP);
        case EXODUS_SURR_HEAVISIDE: EXODUS_KIND(EXODUS_SURR_HEAVISIDE);
        default: return hipErrorInvalidValue;
    }
#undef EXODUS_KIND
}

EXODUS_API int exodus_synlif_forward(float *out_spikes, float *out_vmem, float *out_isyn, const float *input,
                                     const float *vmem_post_initial, const float *isyn_initial,
                                     const float *alpha_mem, const float *alpha_syn, const float *membr_subtract,
                                     const float *theta, const float *theta_low, int apply_theta_low,
                                     int max_num_spikes, int decay_early, int norm_input, int64_t n, int64_t t,
                                     void *stream)
{
    if (bad_dims(n, t)) return hipErrorInvalidValue;
    if (n == 0 || t == 0) return hipSuccess;
    if (!out_spikes || !out_vmem || !out_isyn || !input || !vmem_post_initial || !isyn_initial || !alpha_mem ||
        !alpha_syn || !membr_subtract || !theta || (apply_theta_low && !theta_low))
        return hipErrorInvalidValue;
    SynLifFwdOp op;
    op.in[0] = input;
    op.out[0] = out_vmem;
    op.out[1] = out_isyn;
    op.der = out_spikes;
    op.v_init = vmem_post_initial;
    op.i_init = isyn_initial;
    op.alpha_mem = alpha_mem;
    op.alpha_syn = alpha_syn;
    op.c = membr_subtract;
    op.theta = theta;
    op.theta_low = theta_low;
    op.apply_low = apply_theta_low ? 1 : 0;
    op.decay_early = decay_early ? 1 : 0;
    op.norm_input = norm_input ? 1 : 0;
    op.cap = static_cast<unsigned>(max_num_spikes);
    return launch<SynLifFwdOp, EXODUS_TT_1>(op, n, t, stream);
}

EXODUS_API int exodus_synlif_backward(float *grad_input, float *alpha_mem_grad, float *alpha_syn_grad,
                                      float *vmem_init_grad, float *isyn_init_grad, const float *grad_spikes,
                                      const float *grad_vmem, const float *grad_isyn, const float *vmem,
                                      const float *isyn, const float *vmem_post_initial, const float *isyn_initial,
                                      const float *alpha_mem, const float *alpha_syn, const float *membr_subtract,
                                      const float *theta, const float *theta_low, int apply_theta_low,
                                      int max_num_spikes, int decay_early, int norm_input, int surrogate_kind,
                                      float surr_p0, float surr_p1, int64_t n, int64_t t, void *stream)
{
    if (bad_dims(n, t)) return hipErrorInvalidValue;
    if (n == 0 || t == 0) return hipSuccess;
    if (!grad_input || !grad_spikes || !vmem || !isyn || !alpha_mem || !alpha_syn || !membr_subtract || !theta)
        return hipErrorInvalidValue;
    if (apply_theta_low && !theta_low) return hipErrorInvalidValue;
    if (alpha_mem_grad && !vmem_post_initial) return hipErrorInvalidValue;
    if (alpha_syn_grad && !decay_early && !isyn_initial) return hipErrorInvalidValue;
    if ((grad_vmem == nullptr) != (grad_isyn == nullptr)) return hipErrorInvalidValue;   // both or neither
    const bool extra = grad_vmem != nullptr;
#define EXODUS_SYN(K)                                                                                           \
    do {                                                                                                        \
        if (extra)                                                                                              \
            return launch_synlif_bwd<K, true>(grad_input, alpha_mem_grad, alpha_syn_grad, vmem_init_grad,       \
                                              isyn_init_grad, grad_spikes, grad_vmem, grad_isyn, vmem, isyn,    \
                                              vmem_post_initial, isyn_initial, alpha_mem, alpha_syn,            \
                                              membr_subtract, theta, theta_low, apply_theta_low ? 1 : 0,        \
                                              max_num_spikes, decay_early ? 1 : 0, norm_input ? 1 : 0, surr_p0, \
                                              surr_p1, n, t, stream);                                           \
        return launch_synlif_bwd<K, false>(grad_input, alpha_mem_grad, alpha_syn_grad, vmem_init_grad,          \
                                           isyn_init_grad, grad_spikes, grad_vmem, grad_isyn, vmem, isyn,       \
                                           vmem_post_initial, isyn_initial, alpha_mem, alpha_syn,               \
                                           membr_subtract, theta, theta_low, apply_theta_low ? 1 : 0,           \
                                           max_num_spikes, decay_early ? 1 : 0, norm_input ? 1 : 0, surr_p0,    \
                                           surr_p1, n, t, stream);                                              \
    } while (0)
    switch (surrogate_kind) {
        case EXODUS_SURR_SINGLE_EXP: EXODUS_SYN(EXODUS_SURR_SINGLE_EXP);
        case EXODUS_SURR_PERIODIC_EXP: EXODUS_SYN(EXODUS_SURR_PERIODIC_EXP);
        case EXODUS_SURR_HEAVISIDE: EXODUS_SYN(EXODUS_SURR_HEAVISIDE);
        default: return hipErrorInvalidValue;
    }
#undef EXODUS_SYN
}

EXODUS_API int exodus_spike_forward(float *out_spikes, float *vmem, float alpha, float membr_subtract, float theta,
                                    float theta_low, int apply_theta_low, int max_num_spikes, int64_t n, int64_t t,
                                    void *stream)
{
    if (bad_dims(n, t)) return hipErrorInvalidValue;
    if (n == 0 || t == 0) return hipSuccess;
    if (!out_spikes || !vmem) return hipErrorInvalidValue;
    SpikeFwdOp op;
    op.in[0] = vmem;
    op.out[0] = vmem;
    op.der = out_spikes;
    op.alpha = alpha;
    op.c = membr_subtract;
    op.theta = theta;
    op.theta_low = theta_low;
    op.apply_low = apply_theta_low ? 1 : 0;
    op.cap = static_cast<unsigned>(max_num_spikes);           // negative -> no cap
    return launch<SpikeFwdOp, EXODUS_TT_1>(op, n, t, stream);
}

EXODUS_API int exodus_spike_backward(float *input_grad, const float *surr, const float *output_grad,
                                     const float *not_clipped, float alpha, float membr_subtract, int64_t n,
                                     int64_t t, void *stream)
{
    if (bad_dims(n, t)) return hipErrorInvalidValue;
    if (n == 0 || t == 0) return hipSuccess;
    if (!input_grad || !surr || !output_grad || !not_clipped) return hipErrorInvalidValue;
    SpikeBwdOp op;
    op.in[0] = output_grad;
    op.in[1] = surr;
    op.in[2] = not_clipped;
    op.out[0] = input_grad;
    op.alpha = alpha;
    op.c = membr_subtract;
    return launch<SpikeBwdOp, EXODUS_TT_3>(op, n, t, stream);
}

}  // extern "C"
