// Split-K exchange shared by the GEMV kernels: the workgroups that cover different K ranges of one
// 256-column tile meet in a caller-provided workspace and the one that arrives last finishes the
// sum in a fixed order (bitwise reproducible) and writes the bf16 output.
//
// Cross-XCD visibility without cache-wide fences: partials are stored write-through at device
// scope and read back with device-scope loads; the counter is a device-scope atomic.  Every wave
// waits for its own stores to be acknowledged before the barrier, and the counter moves after the
// barrier: that is all the ordering the exchange needs.  (A device-scope fence would write back and
// invalidate the whole L2 once per workgroup: measured ~0.25 us per workgroup, serialised.)
// Counters sit on 64-byte lines of their own; packed together they serialise at the memory side
// (~10 ns per atomic, measured).
//
// What the exchange relies on, instruction by instruction (gfx950):
//   1. a producer's partial sums leave as global stores with the device-scope bit (sc1): they are written
//      through to memory, past its XCD's L2, and a store is only counted as complete (vmcnt) once that
//      write-through has been acknowledged;
//   2. s_waitcnt vmcnt(0) in every wave, then the workgroup barrier: when thread 0 passes the barrier, every
//      partial sum of its workgroup has been acknowledged by memory;
//   3. only then thread 0 issues the device-scope atomic increment, which executes at the memory side, the
//      one place all XCDs share;
//   4. the workgroup that reads ktiles - 1 back knows that every other workgroup's increment, hence by 2
//      every other workgroup's partial sums, reached memory before; its read-back uses device-scope loads
//      (sc1), which do not hit in its own, possibly stale, L1 or L2.
// The compiler keeps 1-3 in order because the wait and the barrier are explicit and the atomics are not
// reordered across them (the workgroup-scope release fence in front of the wait pins the stores above it).
// In the language's memory model this is weaker than a release/acquire pair at agent scope; with such a pair
// the compiler adds a write-back and invalidation of the whole L2 per workgroup (measured: 3 us more on a
// 256-workgroup launch, 27 us on 2000 workgroups).  Because the argument is about this chip, other targets
// are refused below, and tests/test_gpu_exchange_soak.py replays thousands of launches on one workspace.
#ifndef KX_SPLITK_EXCHANGE_H
#define KX_SPLITK_EXCHANGE_H

#include "kx_common.h"

#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "kx_splitk_exchange.h orders its memory operations by gfx950's write-through stores and vmcnt acknowledgements; other targets need release/acquire orderings"
#endif

namespace kx {

constexpr int kTileCols = 256;     // output columns per column tile, one thread each in the exchange
constexpr int kCounterStride = 16; // uint32 slots between counters: one 64-byte line each

// Nothing in the language orders the relaxed loads of a read-back behind the relaxed atomic whose result decides
// that they run; the hardware does (the loads sit behind a branch on that result).  This keeps the compiler from
// moving memory operations across the point as well: no instruction, no cache traffic.
__device__ __forceinline__ void compiler_fence() {
    asm volatile("" ::: "memory");
}

__device__ __forceinline__ void store_agent(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_agent(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The partial sums as a buffer for the read-backs that use buffer loads: the lane's column is one vector
// register shared by every load, a K tile's offset (the same in every lane) a scalar register, so that a load
// costs one instruction and no address arithmetic in the vector unit.  The host keeps the partial sums below
// 4 GiB.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t partials_buffer(float* partials, size_t floats) {
    return __builtin_amdgcn_make_buffer_rsrc(partials, 0, static_cast<int>(static_cast<uint32_t>(floats * sizeof(float))),
                                             0x00020000);
}
// Element `lane_bytes / 4` of the K tile that starts `tile_floats` floats into the buffer, device scope (cache
// policy 16 is the sc1 bit, what load_agent's loads carry).
__device__ __forceinline__ float load_partial(__amdgpu_buffer_rsrc_t rsrc, int lane_bytes, uint32_t tile_floats) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, lane_bytes,
                                                                          static_cast<int>(tile_floats * 4u), 16));
}

// Called by every thread of the workgroup (it contains barriers).  Thread tid < 256 owns tile column
// tid and brings psum[r], its partial sum for activation row m0 + r.  `s_prev` is one uint32 of LDS.
// Returns true, the same in every thread, in the workgroup that ends up with the finished sums
// (in `sum`, for the threads that own a column); the others return false and are done.
template <int ROWS>
__device__ __forceinline__ bool splitk_exchange_sum(const float (&psum)[ROWS], float (&sum)[ROWS], int m0, int M,
                                                    int N, int ct, int kt, int ktiles, int counter_index,
                                                    float* __restrict__ partials,
                                                    uint32_t* __restrict__ counters, uint32_t* s_prev) {
    const int tid = threadIdx.x;
    const int col = ct * kTileCols + tid;
    const bool col_ok = (tid < kTileCols) && (col < N);
    if (ktiles == 1) {
#pragma unroll
        for (int r = 0; r < ROWS; r++) sum[r] = psum[r];
        return true;
    }

    const size_t tstride = static_cast<size_t>(M) * N;  // floats between consecutive K tiles
    if (col_ok) {
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            if (m0 + r < M) {
                store_agent(partials + static_cast<size_t>(kt) * tstride + static_cast<size_t>(m0 + r) * N + col, psum[r]);
            }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    uint32_t* counter = counters + static_cast<size_t>(counter_index) * kCounterStride;
    if (tid == 0) {
        *s_prev = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (*s_prev != static_cast<uint32_t>(ktiles - 1)) return false;
    compiler_fence();  // the read-back below stays behind the counter's return

    // Last to arrive: every other workgroup's partials were acknowledged before its increment.
    // The read-back is a round trip to memory (~1 us, the longest leg of the exchange), so as many
    // loads as the registers allow go out together: TB K-tiles of every row per thread.  Per row the
    // additions keep a fixed order: t = 0, 1, 2, ... or, with helpers, the even tiles in that order,
    // the odd ones likewise, then even + odd.
#pragma unroll
    for (int r = 0; r < ROWS; r++) sum[r] = 0.0f;
    constexpr int TB = ROWS >= 16 ? 4 : 16;
    // One activation row, more K tiles than one batch, and threads to spare: the upper half of a
    // 512-thread workgroup reads the odd tiles, which halves the number of dependent batches.
    const bool helpers = ROWS == 1 && ktiles > TB && blockDim.x >= 2 * kTileCols;
    const int lane_col = tid % kTileCols;
    // 0: the column's owner, 1: its helper; the same for a whole wave, and said so to the compiler,
    // which then keeps the K-tile offsets in scalar registers (one vector register of addresses
    // instead of two per load in flight)
    const int half = __builtin_amdgcn_readfirstlane(tid / kTileCols);
    const unsigned hcol = static_cast<unsigned>(ct * kTileCols + lane_col);
    const int step = helpers ? 2 : 1;
    if ((helpers ? half < 2 : tid < kTileCols) && hcol < static_cast<unsigned>(N)) {
        for (int t0 = helpers ? half : 0; t0 < ktiles; t0 += TB * step) {
            float v[ROWS][TB];
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
#pragma unroll
                for (int u = 0; u < TB; u++) {
                    // clamped address, masked value: the loads of a batch are straight-line code
                    const int t = t0 + u * step;
                    const int tc = t < ktiles ? t : ktiles - 1;
                    const int mc = m0 + r < M ? m0 + r : M - 1;
                    const float* row = partials + static_cast<size_t>(tc) * tstride + static_cast<size_t>(mc) * N;
                    const float got = load_agent(row + hcol);
                    v[r][u] = (m0 + r < M && t < ktiles) ? got : 0.0f;
                }
            }
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
#pragma unroll
                for (int u = 0; u < TB; u++) sum[r] += v[r][u];
            }
        }
    }
    if (helpers) {
        __shared__ float s_help[kTileCols];
        if (half == 1) s_help[lane_col] = sum[0];
        __syncthreads();
        if (half == 0) sum[0] += s_help[lane_col];
    }
    if (tid == 0) {
        // leave the workspace ready for the next launch
        __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return true;
}

// The exchange followed by the plain epilogue: y[m, col] = bf16(sum).
template <int ROWS>
__device__ __forceinline__ void splitk_exchange_store(const float (&psum)[ROWS], int m0, int M, int N,
                                                      int ct, int kt, int ktiles, int counter_index,
                                                      float* __restrict__ partials,
                                                      uint32_t* __restrict__ counters,
                                                      uint16_t* __restrict__ y, uint32_t* s_prev) {
    float sum[ROWS];
    if (!splitk_exchange_sum<ROWS>(psum, sum, m0, M, N, ct, kt, ktiles, counter_index, partials, counters, s_prev)) {
        return;
    }
    const int col = ct * kTileCols + static_cast<int>(threadIdx.x);
    if (threadIdx.x < kTileCols && col < N) {
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            if (m0 + r < M) y[static_cast<size_t>(m0 + r) * N + col] = f32_to_bf16(sum[r]);
        }
    }
}

// One activation row and the plain epilogue: every wave of 64 columns is an exchange of its own, with an
// arrival counter per tile quarter (lines kCountersPerTile * tile + quarter of the counter area).  The
// wave waits for its own stores, bumps its counter and, if it is the last of its quarter, reads the
// quarter's partial sums back: no workgroup barrier, no broadcast through LDS, and no wave waits for the
// slowest wave of its workgroup.  The ordering argument is that of the header, per wave instead of per
// workgroup (a wave's atomic is issued after the wave's own stores have been acknowledged).  Per column
// the additions run exactly as in splitk_exchange_sum - K tiles in order, or, where that routine would
// use helper threads (more than sixteen K tiles in a workgroup of at least 512 threads), the even tiles in
// order, the odd ones likewise, then even + odd - so that a plain launch returns the bits of the launches
// whose epilogues go through splitk_exchange_sum.  Measured against the workgroup-wide exchange on the seven
// Qwen3-8B projections: 0.3-0.4 us per launch, 5.5 % on the step.
// Called by every thread; `psum` as in splitk_exchange_sum (thread tid < 256 owns tile column tid).
//
// Returns true, the same in every lane of the wave, in the wave that ends up with the finished sums of its
// 64 columns (`sum`); the other waves return false and are done.  Waves past the tile's 256 columns return
// false at once.
__device__ __forceinline__ bool splitk_exchange_sum_per_wave(float psum, float* sum_out, int N, int ct, int kt,
                                                             int ktiles, int counter_index,
                                                             float* __restrict__ partials,
                                                             uint32_t* __restrict__ counters) {
    const int tid = threadIdx.x;
    if (tid >= kTileCols) return false;  // whole waves: the others own no column
    if (ktiles == 1) {
        *sum_out = psum;
        return true;
    }
    const int col = ct * kTileCols + tid;
    const bool col_ok = col < N;
    const size_t tstride = static_cast<size_t>(N);  // floats between consecutive K tiles: one activation row
    if (col_ok) store_agent(partials + static_cast<size_t>(kt) * tstride + col, psum);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    uint32_t* counter = counters + (static_cast<size_t>(counter_index) * kCountersPerTile + tid / kWave) * kCounterStride;
    uint32_t prev = 0;
    if (tid % kWave == 0) prev = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    prev = __builtin_amdgcn_readfirstlane(prev);
    compiler_fence();  // the read-back below stays behind the counter's return
    if (prev != static_cast<uint32_t>(ktiles - 1)) return false;

    // last of its quarter: every other wave's partial sums were acknowledged before its increment
    constexpr int TB = 16;
    const int lane_bytes = (col_ok ? col : N - 1) * static_cast<int>(sizeof(float));
    const __amdgpu_buffer_rsrc_t rsrc = partials_buffer(partials, static_cast<size_t>(ktiles) * tstride);
    const uint32_t tfloats = static_cast<uint32_t>(N);  // floats between consecutive K tiles
    float sum = 0.0f;
    if (!(ktiles > TB && blockDim.x >= 2 * kTileCols)) {
        for (int t0 = 0; t0 < ktiles; t0 += TB) {
            float v[TB];
#pragma unroll
            for (int u = 0; u < TB; u++) {
                // clamped address, masked value: the loads of a batch are straight-line code
                const int t = t0 + u;
                const int tc = t < ktiles ? t : ktiles - 1;
                const float got = load_partial(rsrc, lane_bytes, static_cast<uint32_t>(tc) * tfloats);
                v[u] = t < ktiles ? got : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < TB; u++) sum += v[u];
        }
    } else {
        // where splitk_exchange_sum has helper threads: the even tiles in order, the odd ones likewise, even + odd.
        // Both runs are in flight together (thirty-two loads per batch).
        float odd = 0.0f;
        for (int t0 = 0; t0 < ktiles; t0 += 2 * TB) {
            // the even run is requested first: its additions start while the odd run is still arriving
            float ve[TB], vo[TB];
#pragma unroll
            for (int u = 0; u < TB; u++) {
                const int t = t0 + 2 * u;
                const int tc = t < ktiles ? t : ktiles - 1;
                const float got = load_partial(rsrc, lane_bytes, static_cast<uint32_t>(tc) * tfloats);
                ve[u] = t < ktiles ? got : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < TB; u++) {
                const int t = t0 + 2 * u + 1;
                const int tc = t < ktiles ? t : ktiles - 1;
                const float got = load_partial(rsrc, lane_bytes, static_cast<uint32_t>(tc) * tfloats);
                vo[u] = t < ktiles ? got : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < TB; u++) sum += ve[u];
#pragma unroll
            for (int u = 0; u < TB; u++) odd += vo[u];
        }
        sum += odd;
    }
    *sum_out = sum;
    if (tid % kWave == 0) {
        // leave the workspace ready for the next launch
        __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return true;
}

// The per-wave exchange followed by the plain epilogue: y[col] = bf16(sum).
__device__ __forceinline__ void splitk_exchange_store_per_wave(float psum, int N, int ct, int kt, int ktiles,
                                                               int counter_index, float* __restrict__ partials,
                                                               uint32_t* __restrict__ counters,
                                                               uint16_t* __restrict__ y) {
    float sum;
    if (!splitk_exchange_sum_per_wave(psum, &sum, N, ct, kt, ktiles, counter_index, partials, counters)) return;
    const int col = ct * kTileCols + static_cast<int>(threadIdx.x);
    if (col < N) store_result(y + col, f32_to_bf16(sum));
}

// ---- One activation row, plain store: the K tiles of a column meet in one 64-bit word ----
//
// Every workgroup turns its partial sum of a column into a 52-bit fixed-point number and adds it to the column's
// slot with one returning device-scope atomic; the slot's top bits count the arrivals, and the thread whose
// atomic returns ktiles - 1 holds, in the returned word plus its own addend, the finished sum: it converts,
// stores y and clears the slot.  One trip to memory where the exchanges above take three (store
// acknowledgement, counter, read-back), and nothing to order: the sum travels in the atomic itself.  Integer
// addition commutes, so the result does not depend on the order of arrival (bitwise reproducible).
//
// slot = [ arrivals : 6 ][ arrivals that took the slow path : 6 ][ sum of (v + 2^45) : 52 ],  |v| < 2^45
//
// The unit of v must be the same in every workgroup of a column and is therefore a function of operands that
// all of them can read: unit = 2^ceil(log2(16 * 256 * sum_k |x[k]| * |scales[0, col]|)) / 2^45, i.e. a
// partial sum fits as long as the scales of its own groups stay below 256 times the column's scale in group 0
// (|q - z| <= 15, the partial's share of sum |x| <= all of it).  A partial sum of typical magnitude keeps
// 29 bits, more than its fp32 mantissa; in general the exchange adds at most ktiles * unit / 2 to a column.
// A partial sum that does not fit (far larger scales than group 0's, or not finite) takes the slow path: it is
// left as fp32 in `partials` (as in the exchanges above), its K tile is marked in the column's mask word, and
// only then the slot is bumped, with the slow-path count; the finishing thread then adds the marked partial
// sums in K-tile order, in double.  Slots and masks live in the zeroed area that otherwise holds the arrival
// counters (N * 16 bytes) and are left zeroed.
constexpr int kFixedCountShift = 58;
constexpr int kFixedSlowShift = 52;
constexpr int kFixedBiasLog2 = 45;
constexpr int kFixedMaxKTiles = 63;   // arrivals must fit six bits, K tiles the 64-bit mask

struct FixedUnit {
    float unit, inv_unit;  // powers of two
};

// `ref` = sum |x| * |scales[0, col]| >= 0 (or NaN / Inf, which take the largest unit).
__device__ __forceinline__ FixedUnit fixed_unit_of(float ref) {
    int e = static_cast<int>((__float_as_uint(ref) >> 23) & 0xffu);  // ref < 2^(e - 126)
    e = e < 33 ? 33 : (e > 254 ? 254 : e);
    // 2^45 units = 2^(e - 126) * 16 * 256
    FixedUnit u;
    u.unit = __uint_as_float(static_cast<uint32_t>(e - 32) << 23);
    u.inv_unit = __uint_as_float(static_cast<uint32_t>(286 - e) << 23);
    return u;
}

// Called by the threads that own a column (tid < 256), more than one K tile.  `slots` is the zeroed area.
__device__ __forceinline__ void splitk_exchange_store_fixed(float psum, FixedUnit u, int N, int ct, int kt, int ktiles,
                                                            unsigned long long* __restrict__ slots,
                                                            float* __restrict__ partials,
                                                            uint16_t* __restrict__ y) {
    const int col = ct * kTileCols + static_cast<int>(threadIdx.x);
    if (col >= N) return;
    unsigned long long* slot = slots + col;
    unsigned long long* mask = slots + N + col;
    const float t = psum * u.inv_unit;  // exact: a power of two, and what underflows is below the unit
    const bool fits = __builtin_fabsf(t) < 0x1p45f;  // false for NaN and for a product that overflowed
    // t = hi * 2^24 + lo with |hi| < 2^21 and |lo| <= 2^23, both integers after rounding (garbage, unused, if !fits)
    const float hi = __builtin_rintf(t * 0x1p-24f);
    const float lo = __builtin_fmaf(hi, -0x1p24f, t);  // exact
    const long long v = (static_cast<long long>(static_cast<int>(hi)) << 24) +
                        static_cast<long long>(static_cast<int>(__builtin_rintf(lo)));
    unsigned long long add = (1ull << kFixedCountShift) + static_cast<unsigned long long>(v + (1ll << kFixedBiasLog2));
    if (__builtin_expect(!fits, 0)) {
        store_agent(partials + static_cast<size_t>(kt) * N + col, psum);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);
        // returning, so that the wait below covers it: the mark is in memory before the slot moves
        const unsigned long long seen = __hip_atomic_fetch_or(mask, 1ull << kt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("" ::"v"(seen));
        __builtin_amdgcn_s_waitcnt(0);
        add = (1ull << kFixedCountShift) + (1ull << kFixedSlowShift) + (1ull << kFixedBiasLog2);
    }
    const unsigned long long old = __hip_atomic_fetch_add(slot, add, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if ((old >> kFixedCountShift) != static_cast<unsigned long long>(ktiles - 1)) return;
    const unsigned long long total = old + add;
    const long long value = static_cast<long long>(total & ((1ull << kFixedSlowShift) - 1)) -
                            static_cast<long long>(ktiles) * (1ll << kFixedBiasLog2);
    double sum = static_cast<double>(value) * static_cast<double>(u.unit);
    if (__builtin_expect(((total >> kFixedSlowShift) & 63ull) != 0, 0)) {
        const unsigned long long m = __hip_atomic_load(mask, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int tt = 0; tt < ktiles; tt++) {
            if ((m >> tt) & 1ull) sum += static_cast<double>(load_agent(partials + static_cast<size_t>(tt) * N + col));
        }
        __hip_atomic_store(mask, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    store_result(y + col, f32_to_bf16(static_cast<float>(sum)));
    __hip_atomic_store(slot, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The per-wave exchange for ROWS activation rows (M <= ROWS of them live) of a workgroup of 256 threads:
// partial sums laid out [K tile][M][N] as in splitk_exchange_sum, one arrival counter per wave of 64 columns,
// the last wave of a quarter reads every row of its columns back, K tiles in order (the order of
// splitk_exchange_sum without helper threads, so the bits are those of that routine).
// Returns true, the same in every lane, in the wave that ends up with the finished sums (`sum`, rows at or
// past M are zero); the other waves return false and are done.
template <int ROWS>
__device__ __forceinline__ bool splitk_exchange_sum_per_wave_rows(const float (&psum)[ROWS], float (&sum)[ROWS], int M,
                                                                  int N, int ct, int kt, int ktiles,
                                                                  float* __restrict__ partials,
                                                                  uint32_t* __restrict__ counters) {
    static_assert(ROWS >= 1 && ROWS <= 4, "sixteen K tiles of every row are in flight together");
    const int tid = threadIdx.x;
    if (tid >= kTileCols) return false;  // whole waves: the others own no column
    if (ktiles == 1) {
#pragma unroll
        for (int r = 0; r < ROWS; r++) sum[r] = r < M ? psum[r] : 0.0f;
        return true;
    }
    const int col = ct * kTileCols + tid;
    const bool col_ok = col < N;
    const size_t tstride = static_cast<size_t>(M) * N;  // floats between consecutive K tiles
    if (col_ok) {
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            if (r < M) store_agent(partials + static_cast<size_t>(kt) * tstride + static_cast<size_t>(r) * N + col, psum[r]);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    uint32_t* counter = counters + (static_cast<size_t>(ct) * kCountersPerTile + tid / kWave) * kCounterStride;
    uint32_t prev = 0;
    if (tid % kWave == 0) prev = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    prev = __builtin_amdgcn_readfirstlane(prev);
    compiler_fence();  // the read-back below stays behind the counter's return
    if (prev != static_cast<uint32_t>(ktiles - 1)) return false;

    // last of its quarter: every other wave's partial sums were acknowledged before its increment
    constexpr int TB = 16;
    const int lane_bytes = (col_ok ? col : N - 1) * static_cast<int>(sizeof(float));
    const __amdgpu_buffer_rsrc_t rsrc = partials_buffer(partials, static_cast<size_t>(ktiles) * tstride);
    const uint32_t tfloats = static_cast<uint32_t>(tstride);
#pragma unroll
    for (int r = 0; r < ROWS; r++) sum[r] = 0.0f;
    for (int t0 = 0; t0 < ktiles; t0 += TB) {
        float v[ROWS][TB];
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
#pragma unroll
            for (int u = 0; u < TB; u++) {
                // clamped address, masked value: the loads of a batch are straight-line code
                const int t = t0 + u;
                const int tc = t < ktiles ? t : ktiles - 1;
                const int rc = r < M ? r : M - 1;
                const float got = load_partial(rsrc, lane_bytes, static_cast<uint32_t>(tc) * tfloats +
                                                                     static_cast<uint32_t>(rc) * static_cast<uint32_t>(N));
                v[r][u] = (t < ktiles && r < M) ? got : 0.0f;
            }
        }
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
#pragma unroll
            for (int u = 0; u < TB; u++) sum[r] += v[r][u];
        }
    }
    if (tid % kWave == 0) {
        // leave the workspace ready for the next launch
        __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return true;
}

// Sums of the partial sums of columns `col` and `col + 64` over K tiles t_begin, t_begin + STEP, ... below
// `ktiles`, added to `a` and `b` in that order; batches of sixteen K tiles (thirty-two loads in flight) with
// clamped addresses and masked values, straight-line code per batch.
template <int STEP>
__device__ __forceinline__ void splitk_column_pair_run(__amdgpu_buffer_rsrc_t rsrc, uint32_t tfloats,
                                                       unsigned col, int t_begin, int ktiles, float* a, float* b) {
    constexpr int TB = 16;
    float sa = *a, sb = *b;
    for (int t0 = t_begin; t0 < ktiles; t0 += STEP * TB) {
        float va[TB], vb[TB];
#pragma unroll
        for (int u = 0; u < TB; u++) {
            const int t = t0 + STEP * u;
            const int tc = t < ktiles ? t : ktiles - 1;
            const float ga = load_partial(rsrc, static_cast<int>(col * sizeof(float)), static_cast<uint32_t>(tc) * tfloats);
            const float gb = load_partial(rsrc, static_cast<int>((col + kWave) * sizeof(float)), static_cast<uint32_t>(tc) * tfloats);
            va[u] = t < ktiles ? ga : 0.0f;
            vb[u] = t < ktiles ? gb : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < TB; u++) {
            sa += va[u];
            sb += vb[u];
        }
    }
    *a = sa;
    *b = sb;
}

// One activation row, more than one K tile, and an epilogue that works on heads of 128 columns (two waves of
// the tile): the two waves of a head share an arrival counter (lines kCountersPerTile * tile + 2 * (head in
// tile)), every wave reports for itself as in splitk_exchange_sum_per_wave, and the last of the head's
// 2 * ktiles waves reads both halves back: lane i ends up with columns i (`lo`) and i + 64 (`hi`) of the
// head, the layout of the rotary routine.  Per column the additions run as in splitk_exchange_sum.
// Returns true, the same in every lane, in that last wave; every other wave returns false and is done.
// N is a multiple of 256 here (whole tiles of two heads).
__device__ __forceinline__ bool splitk_exchange_sum_per_head(float psum, float* lo, float* hi, int N, int ct, int kt,
                                                             int ktiles, float* __restrict__ partials,
                                                             uint32_t* __restrict__ counters) {
    const int tid = threadIdx.x;
    if (tid >= kTileCols) return false;  // whole waves: the others own no column
    const int col = ct * kTileCols + tid;
    const size_t tstride = static_cast<size_t>(N);
    store_agent(partials + static_cast<size_t>(kt) * tstride + col, psum);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    const int head_in_tile = tid / (2 * kWave);
    uint32_t* counter = counters + (static_cast<size_t>(ct) * kCountersPerTile + 2 * head_in_tile) * kCounterStride;
    uint32_t prev = 0;
    if (tid % kWave == 0) prev = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    prev = __builtin_amdgcn_readfirstlane(prev);
    compiler_fence();  // the read-back below stays behind the counter's return
    if (prev != static_cast<uint32_t>(2 * ktiles - 1)) return false;

    // last of its head: every other wave's partial sums were acknowledged before its increment
    const int first = ct * kTileCols + head_in_tile * 2 * kWave + tid % kWave;
    const __amdgpu_buffer_rsrc_t rsrc = partials_buffer(partials, static_cast<size_t>(ktiles) * tstride);
    const uint32_t tfloats = static_cast<uint32_t>(N);  // floats between consecutive K tiles
    float a = 0.0f, b = 0.0f;
    if (!(ktiles > 16 && blockDim.x >= 2 * kTileCols)) {
        splitk_column_pair_run<1>(rsrc, tfloats, static_cast<unsigned>(first), 0, ktiles, &a, &b);
    } else {
        // where splitk_exchange_sum has helper threads: the even tiles in order, the odd ones likewise, even + odd
        float ao = 0.0f, bo = 0.0f;
        splitk_column_pair_run<2>(rsrc, tfloats, static_cast<unsigned>(first), 0, ktiles, &a, &b);
        splitk_column_pair_run<2>(rsrc, tfloats, static_cast<unsigned>(first), 1, ktiles, &ao, &bo);
        a += ao;
        b += bo;
    }
    *lo = a;
    *hi = b;
    if (tid % kWave == 0) {
        // leave the workspace ready for the next launch
        __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return true;
}

// The exchange for several activation rows (ROWS = 4, 8 or 16) and a workgroup of exactly 256 threads, more
// than one K tile.  Partial sums go out as above, one column per thread.  The last workgroup reads them back
// two columns per load: threads 0..127 take rows 0 .. ROWS/2-1 of column pairs 0..127, threads 128..255 the
// other rows, so a K tile costs a thread ROWS/2 eight-byte loads instead of ROWS four-byte ones and every
// K tile of the usual shapes is in flight at once.  Per output the additions run t = 0, 1, 2, ... as in
// the narrow exchange.
// Returns true, the same in every thread, in the workgroup that ends up with the finished sums: thread tid
// then holds rows (tid / 128) * ROWS/2 + i, i < ROWS/2, of columns 2 (tid % 128) (`lo`) and the next one
// (`hi`) of the tile.  `before_read_back()` runs in that workgroup once it knows it is the last one, ahead
// of the read-back: loads issued there return under the read-back's round trip.
template <int ROWS, class Before>
__device__ __forceinline__ bool splitk_exchange_sum_wide(const float (&psum)[ROWS], float (&lo)[ROWS / 2],
                                                         float (&hi)[ROWS / 2], int M, int N, int ct, int kt,
                                                         int ktiles, float* __restrict__ partials,
                                                         uint32_t* __restrict__ counters, uint32_t* s_prev,
                                                         Before&& before_read_back) {
    static_assert(ROWS == 4 || ROWS == 8 || ROWS == 16, "row counts the wide read-back is laid out for");
    const int tid = threadIdx.x;
    const int col = ct * kTileCols + tid;
    const size_t tstride = static_cast<size_t>(M) * N;
    if (col < N) {
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            if (r < M) store_agent(partials + static_cast<size_t>(kt) * tstride + static_cast<size_t>(r) * N + col, psum[r]);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    uint32_t* counter = counters + static_cast<size_t>(ct) * kCounterStride;
    if (tid == 0) {
        *s_prev = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (*s_prev != static_cast<uint32_t>(ktiles - 1)) return false;
    compiler_fence();  // the read-back below stays behind the counter's return
    before_read_back();

    constexpr int HALF = ROWS / 2;   // rows per thread
    constexpr int TB = HALF >= 4 ? 64 / HALF : 16;  // K tiles per batch: up to 64 loads in flight
    const int row0 = __builtin_amdgcn_readfirstlane(tid / (kTileCols / 2)) * HALF;  // the same for a whole wave
    const unsigned col2 = static_cast<unsigned>(ct * kTileCols + 2 * (tid % (kTileCols / 2)));
    // Buffer loads: the lane's column is one 32-bit register shared by every load, the row's offset
    // (the same in every lane) a scalar register, so a load in flight costs its two data registers
    // and nothing else.  Cache policy 16 is the device-scope bit (sc1), as on the loads above.
    // The host keeps the partial sums below 4 GiB.
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        partials, 0, static_cast<int>(static_cast<uint32_t>(static_cast<size_t>(ktiles) * tstride * sizeof(float))),
        0x00020000);
    constexpr int kDeviceScope = 16;
#pragma unroll
    for (int i = 0; i < HALF; i++) lo[i] = hi[i] = 0.0f;
    if (col2 < static_cast<unsigned>(N)) {  // N is even: a pair is all in or all out
        const int lane_bytes = static_cast<int>(col2 * sizeof(float));
        for (int t0 = 0; t0 < ktiles; t0 += TB) {
            // two scalars per load: a bit cast applied to one element of a vector (v.y) reads
            // element 0 with this compiler
            uint32_t va[HALF][TB], vb[HALF][TB];
#pragma unroll
            for (int i = 0; i < HALF; i++) {
#pragma unroll
                for (int u = 0; u < TB; u++) {
                    // clamped address, masked value: the loads of a batch are straight-line code
                    const int t = t0 + u;
                    const int tc = t < ktiles ? t : ktiles - 1;
                    const int m = row0 + i;
                    const int mc = m < M ? m : M - 1;
                    // M*N and N are multiples of eight: the row starts on an 8-byte boundary
                    const uint32_t row_pairs = static_cast<uint32_t>((static_cast<size_t>(tc) * tstride + static_cast<size_t>(mc) * N) / 2);
                    const u32x2 got = __builtin_amdgcn_raw_buffer_load_b64(rsrc, lane_bytes, static_cast<int>(row_pairs * 8u), kDeviceScope);
                    const bool live = m < M && t < ktiles;
                    va[i][u] = live ? got.x : 0u;  // all-zero bits are +0.0f
                    vb[i][u] = live ? got.y : 0u;
                }
            }
#pragma unroll
            for (int i = 0; i < HALF; i++) {
#pragma unroll
                for (int u = 0; u < TB; u++) {
                    lo[i] += __builtin_bit_cast(float, va[i][u]);
                    hi[i] += __builtin_bit_cast(float, vb[i][u]);
                }
            }
        }
    }
    if (tid == 0) {
        // leave the workspace ready for the next launch
        __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return true;
}

// The wide exchange followed by the plain epilogue: y[m, col] = bf16(sum), two columns per store.
template <int ROWS>
__device__ __forceinline__ void splitk_exchange_store_wide(const float (&psum)[ROWS], int M, int N, int ct, int kt,
                                                           int ktiles, float* __restrict__ partials,
                                                           uint32_t* __restrict__ counters,
                                                           uint16_t* __restrict__ y, uint32_t* s_prev) {
    const int tid = threadIdx.x;
    if (ktiles == 1) {
        const int col = ct * kTileCols + tid;
        if (col < N) {
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                if (r < M) y[static_cast<size_t>(r) * N + col] = f32_to_bf16(psum[r]);
            }
        }
        return;
    }
    constexpr int HALF = ROWS / 2;
    float lo[HALF], hi[HALF];
    if (!splitk_exchange_sum_wide<ROWS>(psum, lo, hi, M, N, ct, kt, ktiles, partials, counters, s_prev, [] {})) return;
    const int row0 = __builtin_amdgcn_readfirstlane(tid / (kTileCols / 2)) * HALF;
    const unsigned col2 = static_cast<unsigned>(ct * kTileCols + 2 * (tid % (kTileCols / 2)));
    if (col2 < static_cast<unsigned>(N)) {
#pragma unroll
        for (int i = 0; i < HALF; i++) {
            const int m = row0 + i;
            if (m < M) {
                *reinterpret_cast<uint32_t*>(y + static_cast<size_t>(m) * N + col2) = f32x2_to_bf16x2(lo[i], hi[i]);
            }
        }
    }
}

}  // namespace kx

#endif  // KX_SPLITK_EXCHANGE_H
