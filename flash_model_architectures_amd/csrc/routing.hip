// Routing metadata for the MoE layer on gfx950: expert histogram (continuous_count), exclusive
// offsets, stable counting-sort permutation, and the router's top-k + softmax (forward and
// backward).  All integer results are order-independent or explicitly ordered, so they are
// bit-exact from run to run.
//
// Work decomposition of the counting sort: the id stream is cut into contiguous chunks ("units") of
// kChunk ids.  (1) the histogram of every unit is built in LDS and written out as a row of
// `unit_hist[units][E]`; (2) a column-wise exclusive scan over the units plus an exclusive scan
// over the experts turn the rows into the first output slot of every (unit, expert) pair; (3) the
// unit is walked again in order, equal ids inside each 64-wide batch are ranked with ballots, and
// the permutation is written.  For the sizes of an MoE layer a unit belongs to a block of four
// waves (a quarter each) and steps (2) and (3) are one kernel; beyond, a unit belongs to one wave.
#include <mutex>

#include "common.h"

namespace xma {

constexpr int kChunk = 1024;        // ids per unit of the counting sort
constexpr int kMaxExperts = 16384;  // same limit as the reference kernel (forward.cu:12)

// Working memory of xma_route_build_static, the entry point that allocates nothing: the per-chunk histograms
// that xma_route_build keeps in its caller's workspace live here instead.  One copy per GPU, held until the
// process ends; every call on a GPU shares it, so calls that overlap on one GPU race.  Host code never uses the
// array's name as an address: it asks the runtime for the array's device address once per device
// (static_scratch_for_current_device) and passes that pointer to the kernels.
constexpr int64_t kStaticScratchWords = 262144;  // 1 MiB
static __device__ __align__(256) uint32_t scratch[kStaticScratchWords];

// ------------------------------------------------------------------------------------------
// continuous_count
// ------------------------------------------------------------------------------------------
__global__ void fill_u32_kernel(uint32_t* p, int64_t n, uint32_t v) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// LDS holds `copies` replicas of the histogram (stride `bins`); lane l uses replica l % copies,
// which divides the same-address serialisation of LDS atomics when there are few bins.
template <typename IdT>
__global__ __launch_bounds__(256) void count_kernel(const IdT* __restrict__ ids, int64_t n, int bins,
                                                     int copies, int vec_ok, uint32_t* __restrict__ counts) {
    extern __shared__ uint32_t lds_hist[];
    const int total = bins * copies;
    for (int i = threadIdx.x; i < total; i += blockDim.x) lds_hist[i] = 0;
    __syncthreads();

    uint32_t* mine = lds_hist + (threadIdx.x % copies) * bins;
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
    constexpr int kPerVec = 16 / sizeof(IdT);

    if (vec_ok) {
        const int64_t nvec = n / kPerVec;
        const uint4* v = reinterpret_cast<const uint4*>(ids);
        for (int64_t i = tid; i < nvec; i += nthreads) {
            uint4 q = load_stream(v + i);
            IdT e[kPerVec];
            if constexpr (sizeof(IdT) == 4) {
                e[0] = (IdT)q.x;
                e[1] = (IdT)q.y;
                e[2] = (IdT)q.z;
                e[3] = (IdT)q.w;
            } else {
                e[0] = (IdT)(((uint64_t)q.y << 32) | q.x);
                e[1] = (IdT)(((uint64_t)q.w << 32) | q.z);
            }
#pragma unroll
            for (int j = 0; j < kPerVec; ++j)
                if (e[j] >= 0 && e[j] < bins) atomicAdd(&mine[e[j]], 1u);
        }
        for (int64_t i = nvec * kPerVec + tid; i < n; i += nthreads) {
            IdT e = ids[i];
            if (e >= 0 && e < bins) atomicAdd(&mine[e], 1u);
        }
    } else {
        for (int64_t i = tid; i < n; i += nthreads) {
            IdT e = ids[i];
            if (e >= 0 && e < bins) atomicAdd(&mine[e], 1u);
        }
    }
    __syncthreads();

    for (int b = threadIdx.x; b < bins; b += blockDim.x) {
        uint32_t c = 0;
        for (int r = 0; r < copies; ++r) c += lds_hist[r * bins + b];
        if (c) atomicAdd(&counts[b], c);
    }
}

// Small inputs: ONE block builds the whole histogram in LDS (one replica per wave, summed at the end) and writes
// every bin, so the output needs no clearing beforehand and the call is a single launch.
constexpr int64_t kSingleBlockIds = (int64_t)1 << 15;  // most ids a single block is given (two chunks per wave)
constexpr int kSingleBlockBins = 512;                  // most bins (16 replicas of 2 KiB in LDS)
// The one-block counting sort also writes its output through a single compute unit, which moves some tens of bytes
// per clock: beyond this size two launches over many blocks are faster.
constexpr int64_t kSingleBlockSortIds = (int64_t)1 << 12;
template <typename IdT>
__global__ __launch_bounds__(1024) void count_single_block_kernel(const IdT* __restrict__ ids, int64_t n, int bins,
                                                                   uint32_t* __restrict__ counts) {
    extern __shared__ uint32_t lds_hist[];
    constexpr int kWaves = 1024 / kWaveSize;
    for (int i = threadIdx.x; i < bins * kWaves; i += 1024) lds_hist[i] = 0;
    __syncthreads();
    uint32_t* mine = lds_hist + (threadIdx.x / kWaveSize) * bins;
    for (int64_t i = threadIdx.x; i < n; i += 1024) {
        const IdT e = ids[i];
        if (e >= 0 && e < bins) atomicAdd(&mine[e], 1u);
    }
    __syncthreads();
    for (int b = threadIdx.x; b < bins; b += 1024) {
        uint32_t c = 0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) c += lds_hist[w * bins + b];
        counts[b] = c;
    }
}

// ------------------------------------------------------------------------------------------
// stable counting sort
// ------------------------------------------------------------------------------------------
// A wave reads its ids kChunk at a time: 16 per lane, requested together (the walk over a chunk is otherwise a chain
// of dependent load latencies), -1 past `end`.
constexpr int kBatches = kChunk / kWaveSize;
template <typename IdT, int BATCHES>
__device__ __forceinline__ void load_chunk(const IdT* __restrict__ ids, int64_t begin, int64_t end, int lane,
                                           int64_t (&v)[BATCHES]) {
#pragma unroll
    for (int j = 0; j < BATCHES; ++j) {
        const int64_t i = begin + j * kWaveSize + lane;
        v[j] = i < end ? (int64_t)ids[i] : -1;
    }
}

// One 64-wide batch of the placement: lanes holding the same expert id find each other with log2(E) ballots, the
// first of them takes popcount(peers) consecutive slots from next[e], and every lane's slot follows from its rank
// among its peers, so equal ids keep their order.
template <typename OutT>
__device__ __forceinline__ void place_batch(int64_t e64, int64_t i, int E, int nbits, int lane, uint32_t* next,
                                            OutT* __restrict__ sorted_ids, OutT* __restrict__ perm) {
    const bool ok = e64 >= 0 && e64 < E;
    const uint32_t e = ok ? (uint32_t)e64 : 0u;
    uint64_t peers = __ballot(ok);
    for (int b = 0; b < nbits; ++b) {
        const bool bit = (e >> b) & 1u;
        const uint64_t bal = __ballot(ok && bit);
        peers &= bit ? bal : ~bal;
    }
    uint32_t base = 0;
    const int leader = ok ? (int)__ffsll((unsigned long long)peers) - 1 : lane;
    if (ok && leader == lane) base = atomicAdd(&next[e], (uint32_t)__popcll(peers));  // one LDS round trip, not two
    base = __shfl(base, leader, kWaveSize);
    if (ok) {
        const uint32_t pos = base + (uint32_t)__popcll(peers & (((uint64_t)1 << lane) - 1));
        perm[pos] = (OutT)i;
        sorted_ids[pos] = (OutT)e;
    }
}

template <typename IdT>
__global__ __launch_bounds__(256) void unit_hist_kernel(const IdT* __restrict__ ids, int64_t n, int E,
                                                         int waves_per_block, uint32_t* __restrict__ unit_hist) {
    extern __shared__ uint32_t lds_hist[];
    const int wave = threadIdx.x / kWaveSize;
    const int lane = lane_id();
    uint32_t* mine = lds_hist + wave * E;
    const int64_t unit = (int64_t)blockIdx.x * waves_per_block + wave;
    const int64_t begin = unit * kChunk;
    const int64_t end = begin + kChunk < n ? begin + kChunk : n;
    int64_t v[kBatches];
    load_chunk(ids, begin < n ? begin : n, end, lane, v);  // requested before the LDS row is cleared (all -1 past n)
    for (int i = lane; i < E; i += kWaveSize) mine[i] = 0;
    __syncthreads();
    if (begin < n) {
#pragma unroll
        for (int j = 0; j < kBatches; ++j)
            if (v[j] >= 0 && v[j] < E) atomicAdd(&mine[v[j]], 1u);
    }
    __syncthreads();
    if (begin < n) {
        uint32_t* row = unit_hist + unit * E;
        for (int i = lane; i < E; i += kWaveSize) row[i] = mine[i];
    }
}

// The same table of per-unit histograms, written by one block of four waves per unit: a wave counts a quarter of the
// unit (four batches instead of sixteen in a row), the block adds the four rows up.  First launch of the two-launch
// counting sort.
constexpr int kQuarter = kChunk / 4;                  // ids per wave when four waves share a unit
constexpr int kQuarterBatches = kQuarter / kWaveSize;  // 4
template <typename IdT>
__global__ __launch_bounds__(256) void block_hist_kernel(const IdT* __restrict__ ids, int64_t n, int E,
                                                          uint32_t* __restrict__ unit_hist) {
    extern __shared__ uint32_t lds_hist[];  // [4][E]
    const int wave = threadIdx.x / kWaveSize;
    const int lane = lane_id();
    const int64_t unit = blockIdx.x;
    const int64_t begin = unit * kChunk + wave * kQuarter;
    const int64_t end = begin + kQuarter < n ? begin + kQuarter : n;
    int64_t v[kQuarterBatches];
    load_chunk(ids, begin < n ? begin : n, end, lane, v);  // requested before the LDS rows are cleared (all -1 past n)
    for (int i = threadIdx.x; i < 4 * E; i += 256) lds_hist[i] = 0;
    __syncthreads();
    uint32_t* mine = lds_hist + wave * E;
#pragma unroll
    for (int j = 0; j < kQuarterBatches; ++j)
        if (v[j] >= 0 && v[j] < E) atomicAdd(&mine[v[j]], 1u);
    __syncthreads();
    uint32_t* row = unit_hist + unit * E;
    for (int i = threadIdx.x; i < E; i += 256)
        row[i] = lds_hist[i] + lds_hist[E + i] + lds_hist[2 * E + i] + lds_hist[3 * E + i];
}

// One block of 16 waves per 64 experts: lane = expert column, wave = a segment of the units.
// In place: unit_hist[u][e] becomes the number of ids equal to e in units before u; the column
// totals go to counts[e].
__global__ __launch_bounds__(1024) void unit_scan_kernel(uint32_t* __restrict__ unit_hist, int64_t units, int E,
                                                          uint32_t* __restrict__ counts) {
    __shared__ uint32_t seg_sum[16][kWaveSize];
    const int wave = threadIdx.x / kWaveSize;
    const int lane = lane_id();
    const int e = blockIdx.x * kWaveSize + lane;
    const int64_t seg = (units + 15) / 16;
    const int64_t u0 = wave * seg;
    const int64_t u1 = u0 + seg < units ? u0 + seg : units;
    // both passes keep kScanUnroll independent loads in flight per lane: the column walk is latency-bound
    constexpr int kScanUnroll = 8;
    uint32_t s = 0;
    if (e < E) {
        int64_t u = u0;
        for (; u + kScanUnroll <= u1; u += kScanUnroll) {
            uint32_t v[kScanUnroll];
#pragma unroll
            for (int j = 0; j < kScanUnroll; ++j) v[j] = unit_hist[(u + j) * E + e];
#pragma unroll
            for (int j = 0; j < kScanUnroll; ++j) s += v[j];
        }
        for (; u < u1; ++u) s += unit_hist[u * E + e];
    }
    seg_sum[wave][lane] = s;
    __syncthreads();
    uint32_t base = 0;
    for (int w = 0; w < wave; ++w) base += seg_sum[w][lane];
    if (e < E) {
        int64_t u = u0;
        for (; u + kScanUnroll <= u1; u += kScanUnroll) {
            uint32_t v[kScanUnroll];
#pragma unroll
            for (int j = 0; j < kScanUnroll; ++j) v[j] = unit_hist[(u + j) * E + e];
#pragma unroll
            for (int j = 0; j < kScanUnroll; ++j) {
                unit_hist[(u + j) * E + e] = base;
                base += v[j];
            }
        }
        for (; u < u1; ++u) {
            const uint32_t c = unit_hist[u * E + e];
            unit_hist[u * E + e] = base;
            base += c;
        }
        if (wave == 15) counts[e] = base;
    }
}

// Single block: offsets[0..E] = exclusive scan of counts[0..E).
__global__ __launch_bounds__(1024) void offsets_kernel(const uint32_t* __restrict__ counts, int E,
                                                        int32_t* __restrict__ offsets) {
    __shared__ uint32_t part[1024];
    const int per = (E + 1023) / 1024;  // <= 16
    const int b = threadIdx.x * per;
    uint32_t s = 0;
    for (int i = 0; i < per; ++i)
        if (b + i < E) s += counts[b + i];
    part[threadIdx.x] = s;
    __syncthreads();
    // Hillis-Steele inclusive scan over the 1024 partial sums
    for (int d = 1; d < 1024; d <<= 1) {
        uint32_t v = threadIdx.x >= d ? part[threadIdx.x - d] : 0;
        __syncthreads();
        part[threadIdx.x] += v;
        __syncthreads();
    }
    uint32_t run = part[threadIdx.x] - s;
    for (int i = 0; i < per; ++i) {
        if (b + i < E) {
            offsets[b + i] = (int32_t)run;
            run += counts[b + i];
        }
    }
    if (threadIdx.x == 1023) offsets[E] = (int32_t)part[1023];
}

// offsets[e] = first grouped position whose expert id is >= e, for e in [0, E]: the exclusive prefix sums of the
// histogram, recovered from the sorted ids alone.  Thread p looks at the boundary between positions p - 1 and p
// (position -1 counts as expert -1, position n as expert E) and writes the offsets of the experts that start there,
// so every offsets[e] is written exactly once when the ids are sorted.
template <typename IdT>
__global__ __launch_bounds__(256) void offsets_from_sorted_kernel(const IdT* __restrict__ sorted_ids, int64_t n, int E,
                                                                   int32_t* __restrict__ offsets) {
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p > n) return;
    auto clamped = [&](int64_t i) {
        const int64_t e = (int64_t)sorted_ids[i];
        return e < 0 ? (int64_t)0 : e > E - 1 ? (int64_t)(E - 1) : e;
    };
    const int64_t prev = p == 0 ? -1 : clamped(p - 1);
    const int64_t cur = p == n ? E : clamped(p);
    for (int64_t e = prev + 1; e <= cur; ++e) offsets[e] = (int32_t)p;
}

template <typename IdT, typename OutT>
__global__ __launch_bounds__(256) void place_kernel(const IdT* __restrict__ ids, int64_t n, int E, int nbits,
                                                     int waves_per_block, const uint32_t* __restrict__ unit_prefix,
                                                     const int32_t* __restrict__ offsets, OutT* __restrict__ sorted_ids,
                                                     OutT* __restrict__ perm) {
    extern __shared__ uint32_t lds_hist[];
    const int wave = threadIdx.x / kWaveSize;
    const int lane = lane_id();
    uint32_t* next = lds_hist + wave * E;  // next free output slot per expert, private to this wave
    const int64_t unit = (int64_t)blockIdx.x * waves_per_block + wave;
    const int64_t begin = unit * kChunk;
    if (begin >= n) return;  // no block-wide barrier below, so whole waves may leave
    const uint32_t* row = unit_prefix + unit * E;
    for (int i = lane; i < E; i += kWaveSize) next[i] = row[i] + (uint32_t)offsets[i];
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");

    const int64_t end = begin + kChunk < n ? begin + kChunk : n;
    int64_t v[kBatches];
    load_chunk(ids, begin, end, lane, v);
#pragma unroll
    for (int j = 0; j < kBatches; ++j)
        place_batch(v[j], begin + j * kWaveSize + lane, E, nbits, lane, next, sorted_ids, perm);
}

// The same placement by one block of four waves per unit, a quarter of the unit each (four batches in a row instead
// of sixteen): every wave counts its quarter in LDS, thread e turns column e of the four rows into the first output
// slot of expert e in each quarter, then the waves place their ids.  4 * E words of LDS: for E <= kQuarterMaxExperts.
constexpr int kQuarterMaxExperts = 4096;
template <typename IdT, typename OutT>
__global__ __launch_bounds__(256) void place_quarters_kernel(const IdT* __restrict__ ids, int64_t n, int E, int nbits,
                                                              const uint32_t* __restrict__ unit_prefix,
                                                              const int32_t* __restrict__ offsets,
                                                              OutT* __restrict__ sorted_ids, OutT* __restrict__ perm) {
    extern __shared__ uint32_t lds_hist[];  // [4][E]: a quarter's histogram, then its next free output slots
    const int wave = threadIdx.x / kWaveSize;
    const int lane = lane_id();
    const int64_t unit = blockIdx.x;
    const int64_t begin = unit * kChunk + wave * kQuarter;
    const int64_t end = begin + kQuarter < n ? begin + kQuarter : n;
    int64_t v[kQuarterBatches];
    load_chunk(ids, begin < n ? begin : n, end, lane, v);  // all -1 for a quarter past the end
    // where the unit's ids of expert e start: requested before the first barrier for the first 256 experts
    const uint32_t* row = unit_prefix + unit * E;
    const uint32_t first_start = (int)threadIdx.x < E ? (uint32_t)offsets[threadIdx.x] + row[threadIdx.x] : 0u;
    for (int i = threadIdx.x; i < 4 * E; i += 256) lds_hist[i] = 0;
    __syncthreads();
    uint32_t* next = lds_hist + wave * E;
#pragma unroll
    for (int j = 0; j < kQuarterBatches; ++j)
        if (v[j] >= 0 && v[j] < E) atomicAdd(&next[v[j]], 1u);
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += 256) {
        uint32_t slot = e < 256 ? first_start : (uint32_t)offsets[e] + row[e];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const uint32_t own = lds_hist[w * E + e];
            lds_hist[w * E + e] = slot;
            slot += own;
        }
    }
    __syncthreads();
    if (begin >= n) return;
#pragma unroll
    for (int j = 0; j < kQuarterBatches; ++j)
        place_batch(v[j], begin + j * kWaveSize + lane, E, nbits, lane, next, sorted_ids, perm);
}

// Column sums of the table of per-unit histograms, by one block of 256 threads: total[e] += all units, before[e] +=
// the units before `unit`.  A thread handles V adjacent experts (one 4 * V-byte load per unit) of the units r,
// r + rows, ...; the number of thread columns is E / V rounded up to a power of two, so consecutive lanes read
// consecutive words.  Every load of a thread is requested before the first is used when the table has at most
// kInFlight * rows units.
template <int V>
__device__ __forceinline__ void sum_table(const uint32_t* __restrict__ unit_hist, int64_t units, int64_t unit, int E,
                                          uint32_t* total, uint32_t* before) {
    typedef uint32_t vec_t __attribute__((ext_vector_type(V)));
    constexpr int kInFlight = V == 4 ? 16 : 32;
    const int groups = E / V;
    int cols = 1;
    while (cols < groups) cols <<= 1;
    const int rows = 256 / cols;  // E <= 256
    const int c = threadIdx.x & (cols - 1);
    const int r = threadIdx.x / cols;
    if (c >= groups) return;
    const vec_t* table = reinterpret_cast<const vec_t*>(unit_hist) + c;
    vec_t all = 0, mine = 0;
    for (int64_t u0 = r; u0 < units; u0 += (int64_t)rows * kInFlight) {
        vec_t h[kInFlight];
#pragma unroll
        for (int j = 0; j < kInFlight; ++j) {
            const int64_t u = u0 + (int64_t)j * rows;
            h[j] = u < units ? table[u * groups] : vec_t(0);
        }
#pragma unroll
        for (int j = 0; j < kInFlight; ++j) {
            const int64_t u = u0 + (int64_t)j * rows;
            all += h[j];
            mine += u < unit ? h[j] : vec_t(0);
        }
    }
#pragma unroll
    for (int q = 0; q < V; ++q) {
        atomicAdd(&total[c * V + q], (uint32_t)all[q]);
        atomicAdd(&before[c * V + q], (uint32_t)mine[q]);
    }
}

// Second and last launch of the counting sort for the sizes of an MoE layer (units * E <= kFusedScanValues, E <= 256;
// the first launch is block_hist_kernel).  One work-group moves data at a small fraction of the device's rate, so
// the ids are spread over many small blocks, one unit of four waves each, and every block repeats the scan for
// itself: it reads the whole table of per-unit histograms (at most 64 KiB, L2-resident) and adds up, per expert,
// all units (the expert's total) and the units before its own (where its ids start inside the expert's range);
// thread e scans the totals into the offsets with wave shuffles; then every wave places its quarter of the unit,
// which it requested before the scan began and counted for itself while the table was on its way (a wave's ids
// start after those of the waves before it).  Block 0 also writes counts and offsets.
constexpr int kFusedScanValues = 16384;
template <typename IdT, typename OutT>
__global__ __launch_bounds__(256) void scan_place_kernel(const IdT* __restrict__ ids, int64_t n, int E, int nbits,
                                                          int64_t units, const uint32_t* __restrict__ unit_hist,
                                                          uint32_t* __restrict__ counts, int32_t* __restrict__ offsets,
                                                          OutT* __restrict__ sorted_ids, OutT* __restrict__ perm) {
    extern __shared__ uint32_t lds_hist[];  // total[E], before[E], next[4][E], wave_sum[4]
    uint32_t* total = lds_hist;
    uint32_t* before = lds_hist + E;
    uint32_t* next_all = lds_hist + 2 * E;
    uint32_t* wave_sum = lds_hist + 6 * E;
    const int wave = threadIdx.x / kWaveSize;
    const int lane = lane_id();
    const int64_t unit = blockIdx.x;

    // this wave's ids, on their way while the table is read
    const int64_t begin = unit * kChunk + wave * kQuarter;
    const int64_t end = begin + kQuarter < n ? begin + kQuarter : n;
    int64_t v[kQuarterBatches];
    load_chunk(ids, begin < n ? begin : n, end, lane, v);  // all -1 for a quarter past the end

    for (int i = threadIdx.x; i < 6 * E; i += 256) lds_hist[i] = 0;
    __syncthreads();

    // the wave's own histogram (its quarter of the unit) ...
    {
        uint32_t* own = next_all + wave * E;
#pragma unroll
        for (int j = 0; j < kQuarterBatches; ++j)
            if (v[j] >= 0 && v[j] < E) atomicAdd(&own[v[j]], 1u);
    }
    // ... and the column sums of the table: 16-byte loads when a row is a whole number of them
    if (E % 4 == 0 && (reinterpret_cast<uintptr_t>(unit_hist) & 15) == 0) sum_table<4>(unit_hist, units, unit, E, total, before);
    else sum_table<1>(unit_hist, units, unit, E, total, before);
    __syncthreads();

    // exclusive scan of the totals over the experts: thread e holds expert e
    const int e = threadIdx.x;
    const uint32_t count = e < E ? total[e] : 0u;
    uint32_t inclusive = count;
#pragma unroll
    for (int d = 1; d < kWaveSize; d <<= 1) {
        const uint32_t up = __shfl_up(inclusive, d, kWaveSize);
        if (lane >= d) inclusive += up;
    }
    if (lane == kWaveSize - 1) wave_sum[wave] = inclusive;
    __syncthreads();
    uint32_t first_slot = inclusive - count;
    for (int w = 0; w < wave; ++w) first_slot += wave_sum[w];
    if (e < E) {
        if (blockIdx.x == 0) {
            counts[e] = count;
            offsets[e] = (int32_t)first_slot;
            if (e == E - 1) offsets[E] = (int32_t)(first_slot + count);
        }
        // first output slot of the ids of expert e in each of the block's waves
        uint32_t slot = first_slot + before[e];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const uint32_t own_count = next_all[w * E + e];
            next_all[w * E + e] = slot;
            slot += own_count;
        }
    }
    __syncthreads();

    if (begin >= n) return;
    uint32_t* next = next_all + wave * E;
#pragma unroll
    for (int j = 0; j < kQuarterBatches; ++j)
        place_batch(v[j], begin + j * kWaveSize + lane, E, nbits, lane, next, sorted_ids, perm);
}

// The whole counting sort in ONE block of 16 waves, for up to kSingleBlockSortIds ids and kSingleBlockBins experts (the
// routed rows of a small batch): wave w owns the w-th contiguous run of ids.  (1) every wave builds the histogram
// of its run in its own LDS row; (2) thread e turns column e into exclusive prefixes over the waves, the block
// scans the column totals into the expert offsets, and the two are added up: row w, column e is then the first
// output slot of wave w's ids of expert e; (3) every wave walks its run again in order and ranks equal ids inside
// each 64-wide batch with ballots, as place_kernel does.  No workspace, no other launch.
template <typename IdT, typename OutT>
__global__ __launch_bounds__(1024) void route_single_block_kernel(const IdT* __restrict__ ids, int64_t n, int E,
                                                                   int nbits, uint32_t* __restrict__ counts,
                                                                   int32_t* __restrict__ offsets,
                                                                   OutT* __restrict__ sorted_ids,
                                                                   OutT* __restrict__ perm) {
    extern __shared__ uint32_t lds_hist[];  // [16 waves][E], then [1024] for the scan
    constexpr int kWaves = 1024 / kWaveSize;
    uint32_t* part = lds_hist + kWaves * E;
    const int wave = threadIdx.x / kWaveSize;
    const int lane = lane_id();
    for (int i = threadIdx.x; i < kWaves * E; i += 1024) lds_hist[i] = 0;
    __syncthreads();

    const int64_t per = ((n + kWaves - 1) / kWaves + kWaveSize - 1) / kWaveSize * kWaveSize;  // ids per wave
    const int64_t begin = wave * per < n ? wave * per : n;
    const int64_t end = begin + per < n ? begin + per : n;
    uint32_t* mine = lds_hist + wave * E;
    int64_t v[kBatches];  // the wave's first chunk stays in registers for the placement
    load_chunk(ids, begin, end, lane, v);
#pragma unroll
    for (int j = 0; j < kBatches; ++j)
        if (v[j] >= 0 && v[j] < E) atomicAdd(&mine[v[j]], 1u);
    for (int64_t c0 = begin + kChunk; c0 < end; c0 += kChunk) {
        int64_t u[kBatches];
        load_chunk(ids, c0, end, lane, u);
#pragma unroll
        for (int j = 0; j < kBatches; ++j)
            if (u[j] >= 0 && u[j] < E) atomicAdd(&mine[u[j]], 1u);
    }
    __syncthreads();

    // column e: exclusive prefixes over the waves, total -> counts
    const int e_mine = threadIdx.x;
    uint32_t total = 0;
    if (e_mine < E) {
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const uint32_t c = lds_hist[w * E + e_mine];
            lds_hist[w * E + e_mine] = total;
            total += c;
        }
        counts[e_mine] = total;
    }
    // exclusive scan of the totals over the experts (Hillis-Steele over 1024 slots)
    part[threadIdx.x] = total;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {
        const uint32_t v = threadIdx.x >= d ? part[threadIdx.x - d] : 0;
        __syncthreads();
        part[threadIdx.x] += v;
        __syncthreads();
    }
    const uint32_t first_slot = part[threadIdx.x] - total;
    if (e_mine < E) {
        offsets[e_mine] = (int32_t)first_slot;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) lds_hist[w * E + e_mine] += first_slot;
    }
    if (threadIdx.x == 1023) offsets[E] = (int32_t)part[1023];
    __syncthreads();

    // placement, stable inside the wave's run and across the runs
    uint32_t* next = mine;
#pragma unroll
    for (int j = 0; j < kBatches; ++j)
        place_batch(v[j], begin + j * kWaveSize + lane, E, nbits, lane, next, sorted_ids, perm);
    for (int64_t c0 = begin + kChunk; c0 < end; c0 += kChunk) {
        load_chunk(ids, c0, end, lane, v);
#pragma unroll
        for (int j = 0; j < kBatches; ++j)
            place_batch(v[j], c0 + j * kWaveSize + lane, E, nbits, lane, next, sorted_ids, perm);
    }
}

// ------------------------------------------------------------------------------------------
// router top-k + softmax
// ------------------------------------------------------------------------------------------
// Monotone map float -> uint32 (larger float => larger key); NaN above +inf; -0 == +0.
__device__ __forceinline__ uint32_t order_key(float v) {
    if (v != v) return 0xffffffffu;
    if (v == 0.0f) v = 0.0f;
    uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_to_float(uint32_t key) {
    return __uint_as_float((key & 0x80000000u) ? (key ^ 0x80000000u) : ~key);
}

// Maximum / sum over the aligned group of `width` lanes (a power of two) that the lane belongs to.
__device__ __forceinline__ uint64_t max_with_lane_xor(uint64_t v, int off) {
    uint32_t lo = __shfl_xor((uint32_t)v, off, kWaveSize);
    uint32_t hi = __shfl_xor((uint32_t)(v >> 32), off, kWaveSize);
    uint64_t o = ((uint64_t)hi << 32) | lo;
    return o > v ? o : v;
}
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
#pragma unroll
    for (int off = kWaveSize / 2; off > 0; off >>= 1) v = max_with_lane_xor(v, off);
    return v;
}
__device__ __forceinline__ uint64_t group_max_u64(uint64_t v, int width) {
    if (width == kWaveSize) return wave_max_u64(v);  // constant lane offsets
    for (int off = width / 2; off > 0; off >>= 1) v = max_with_lane_xor(v, off);
    return v;
}
__device__ __forceinline__ float group_sum(float v, int width) {
    for (int off = width / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWaveSize);
    return v;
}

// A group of G lanes per token (G a power of two, k <= G, E <= G * EPL), 64 / G tokens per wave; lane g of the group
// owns experts g, g + G, ...  A round costs EPL compare-and-selects per lane and log2(G) exchange steps, so few lanes
// with many experts each are cheaper than a whole wave per token (E = 64: 8 lanes x 8 experts).
// key = (order_key(value) << 32) | (0xffffffff - expert): the maximum picks the largest value
// and, among equals, the lowest expert index.
template <typename T, int EPL, typename IdxT>
__global__ __launch_bounds__(256) void topk_softmax_kernel(const T* __restrict__ logits, int64_t Tn, int E, int k, int G,
                                                            int64_t ld, T* __restrict__ weights,
                                                            IdxT* __restrict__ idx) {
    const int lane = lane_id();
    const int g = lane & (G - 1);
    const int tokens_per_wave = kWaveSize / G;
    const int64_t first = ((int64_t)blockIdx.x * (blockDim.x / kWaveSize) + threadIdx.x / kWaveSize) * tokens_per_wave;
    if (first >= Tn) return;  // whole waves only: every lane of a wave takes part in the exchanges
    const int64_t t = first + lane / G;
    const bool live = t < Tn;
    const T* row = logits + (live ? t : first) * ld;
    uint64_t keys[EPL];
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
        const int e = g + j * G;
        keys[j] = e < E ? (((uint64_t)order_key(Elem<T>::load(row + e)) << 32) | (uint32_t)(0xffffffffu - (uint32_t)e))
                        : 0ull;
    }
    float my_val = 0.0f;
    uint32_t my_idx = 0;
    float vmax = 0.0f;
    for (int s = 0; s < k; ++s) {
        uint64_t best = 0;
#pragma unroll
        for (int j = 0; j < EPL; ++j) best = keys[j] > best ? keys[j] : best;
        best = group_max_u64(best, G);
#pragma unroll
        for (int j = 0; j < EPL; ++j)
            if (keys[j] == best) keys[j] = 0ull;
        const float v = key_to_float((uint32_t)(best >> 32));
        if (s == 0) vmax = v;
        if (g == s) {
            my_val = v;
            my_idx = 0xffffffffu - (uint32_t)best;
        }
    }
    const float ex = g < k ? expf(my_val - vmax) : 0.0f;
    const float denom = group_sum(ex, G);
    if (live && g < k) {
        Elem<T>::store(weights + t * k + g, ex / denom);
        idx[t * k + g] = (IdxT)my_idx;
    }
}

// Any E <= 16384: one wave per block, ordered keys of the row staged in LDS.
template <typename T, typename IdxT>
__global__ __launch_bounds__(64) void topk_softmax_lds_kernel(const T* __restrict__ logits, int64_t Tn, int E, int k,
                                                               int64_t ld, T* __restrict__ weights,
                                                               IdxT* __restrict__ idx) {
    extern __shared__ uint32_t lds_keys[];
    const int lane = lane_id();
    const int64_t t = blockIdx.x;
    const T* row = logits + t * ld;
    for (int e = lane; e < E; e += kWaveSize) lds_keys[e] = order_key(Elem<T>::load(row + e));
    __syncthreads();
    float my_val = 0.0f, vmax = 0.0f;
    uint32_t my_idx = 0;
    for (int s = 0; s < k; ++s) {
        uint64_t best = 0;
        for (int e = lane; e < E; e += kWaveSize) {
            const uint32_t kk = lds_keys[e];
            // order_key never returns 0 (its minimum, for -inf, is 0x007fffff): 0 marks a taken slot
            uint64_t key = ((uint64_t)kk << 32) | (uint32_t)(0xffffffffu - (uint32_t)e);
            if (kk == 0u) key = 0ull;
            best = key > best ? key : best;
        }
        best = wave_max_u64(best);
        const uint32_t win = 0xffffffffu - (uint32_t)best;
        if (lane == 0 && best != 0ull) lds_keys[win] = 0u;
        __syncthreads();
        const float v = key_to_float((uint32_t)(best >> 32));
        if (s == 0) vmax = v;
        if (lane == s) {
            my_val = v;
            my_idx = win;
        }
    }
    const float ex = lane < k ? expf(my_val - vmax) : 0.0f;
    const float denom = wave_sum(ex);
    if (lane < k) {
        Elem<T>::store(weights + t * k + lane, ex / denom);
        idx[t * k + lane] = (IdxT)my_idx;
    }
}

// d_logits[t, :] = 0, then d_logits[t, idx[t, j]] = w_j * (dw_j - sum_i w_i dw_i) with
// w = softmax(logits[t, idx[t, :]]) recomputed in fp32.  A group of G lanes per token (a power of two, k <= G).
template <typename T, typename IdxT>
__global__ __launch_bounds__(256) void topk_softmax_bwd_kernel(const T* __restrict__ logits, int64_t ld_logits,
                                                                const T* __restrict__ d_weights,
                                                                const IdxT* __restrict__ idx, int64_t Tn, int E, int k,
                                                                int G, T* __restrict__ d_logits, int64_t ld) {
    const int lane = lane_id();
    const int g = lane & (G - 1);
    const int64_t first = ((int64_t)blockIdx.x * (blockDim.x / kWaveSize) + threadIdx.x / kWaveSize) * (kWaveSize / G);
    if (first >= Tn) return;  // whole waves only: every lane of a wave takes part in the exchanges
    const int64_t t = first + lane / G;
    const bool live = t < Tn;
    T* out = d_logits + (live ? t : first) * ld;
    if (live)
        for (int e = g; e < E; e += G) Elem<T>::store(out + e, 0.0f);
    int64_t e_sel = 0;
    float v = -INFINITY, dw = 0.0f;
    if (live && g < k) {
        e_sel = (int64_t)idx[t * k + g];
        v = Elem<T>::load(logits + t * ld_logits + e_sel);
        dw = Elem<T>::load(d_weights + t * k + g);
    }
    float vmax = v;
    for (int off = G / 2; off > 0; off >>= 1) vmax = fmaxf(vmax, __shfl_xor(vmax, off, kWaveSize));
    const float ex = live && g < k ? expf(v - vmax) : 0.0f;
    const float w = ex / group_sum(ex, G);
    const float dot = group_sum(w * dw, G);
    // the zero fill above and this store touch the same addresses from different lanes
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (live && g < k) Elem<T>::store(out + e_sel, w * (dw - dot));
}

static int ceil_log2(int v) {
    int b = 0;
    while ((1 << b) < v) ++b;
    return b;
}

static int sort_waves_per_block(int E) {
    int w = 16384 / E;  // 64 KiB of LDS histograms per block
    if (w > 4) w = 4;
    if (w < 1) w = 1;
    return w;
}

// Device address of `scratch` on the GPU that is current for the calling thread; looked up once per device
// (each GPU holds its own copy of the array at its own address).  nullptr + error text on failure.
static uint32_t* static_scratch_for_current_device() {
    constexpr int kMaxDevices = 64;
    static std::mutex lock;
    static uint32_t* address[kMaxDevices] = {};
    int device = -1;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess || device < 0 || device >= kMaxDevices) {
        set_error("xma_route_build_static: no usable current device (%s, device %d)", hipGetErrorString(err), device);
        return nullptr;
    }
    std::lock_guard<std::mutex> guard(lock);
    if (address[device] == nullptr) {
        void* p = nullptr;
        err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (err != hipSuccess || p == nullptr) {
            set_error("xma_route_build_static: hipGetSymbolAddress failed on device %d: %s", device,
                      hipGetErrorString(err));
            return nullptr;
        }
        address[device] = static_cast<uint32_t*>(p);
    }
    return address[device];
}

}  // namespace xma

using namespace xma;

extern "C" {

int xma_continuous_count(const void* ids, int ids_is_i64, int64_t n, int32_t bins, uint32_t* counts,
                         void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    XMA_REQUIRE(bins >= 1 && bins <= kMaxExperts, "xma_continuous_count: bins=%d outside [1, %d]", bins, kMaxExperts);
    XMA_REQUIRE(n >= 0 && n < ((int64_t)1 << 32), "xma_continuous_count: n=%lld does not fit uint32", (long long)n);
    XMA_REQUIRE(counts != nullptr && (ids != nullptr || n == 0), "xma_continuous_count: null pointer");
    if (n <= kSingleBlockIds && bins <= kSingleBlockBins) {  // one launch, writes every bin
        const size_t lds = (size_t)bins * (1024 / kWaveSize) * sizeof(uint32_t);
        if (ids_is_i64)
            hipLaunchKernelGGL(count_single_block_kernel<int64_t>, dim3(1), dim3(1024), lds, stream, (const int64_t*)ids, n,
                               (int)bins, counts);
        else
            hipLaunchKernelGGL(count_single_block_kernel<int32_t>, dim3(1), dim3(1024), lds, stream, (const int32_t*)ids, n,
                               (int)bins, counts);
        return check_launch("xma_continuous_count");
    }
    hipLaunchKernelGGL(fill_u32_kernel, dim3((bins + 255) / 256), dim3(256), 0, stream, counts, (int64_t)bins, 0u);
    if (n > 0) {
        int copies = 2048 / bins;
        if (copies > 32) copies = 32;
        if (copies < 1) copies = 1;
        // ids per block: every block ends with one global atomic per non-empty bin, all blocks onto the same few
        // lines, so a stream of a million ids is faster over half as many blocks (6.0 against 7.2 us at 2^20 ids,
        // 256 bins), while a short stream needs the blocks (98304 ids: 6.2 against 9.5 us)
        const int per_block = n > ((int64_t)1 << 18) ? 256 * 32 : 256 * 16;
        int64_t blocks = ceil_div(n, per_block);
        if (blocks > 2048) blocks = 2048;
        const size_t lds = (size_t)bins * copies * sizeof(uint32_t);
        const int vec_ok = aligned16(ids) ? 1 : 0;
        if (ids_is_i64)
            hipLaunchKernelGGL(count_kernel<int64_t>, dim3((unsigned)blocks), dim3(256), lds, stream,
                               (const int64_t*)ids, n, (int)bins, copies, vec_ok, counts);
        else
            hipLaunchKernelGGL(count_kernel<int32_t>, dim3((unsigned)blocks), dim3(256), lds, stream,
                               (const int32_t*)ids, n, (int)bins, copies, vec_ok, counts);
    }
    return check_launch("xma_continuous_count");
}

int64_t xma_route_workspace_bytes(int64_t n, int32_t num_experts) {
    if (n < 0 || num_experts < 1) return -1;
    const int64_t units = ceil_div(n > 0 ? n : 1, kChunk);
    return units * (int64_t)num_experts * (int64_t)sizeof(uint32_t);
}

// Launches of the counting sort; arguments already validated.  Every word of `workspace` that is read has been
// written by an earlier kernel of the same call, so the workspace needs no clearing.
static int route_build_launch(const void* ids, int ids_is_i64, int64_t n, int32_t E, uint32_t* counts,
                              int32_t* offsets, void* sorted_ids, void* perm, int out_is_i64, void* workspace,
                              hipStream_t stream) {
    if (n == 0) {
        hipLaunchKernelGGL(fill_u32_kernel, dim3((E + 255) / 256), dim3(256), 0, stream, counts, (int64_t)E, 0u);
        hipLaunchKernelGGL(fill_u32_kernel, dim3((E + 1 + 255) / 256), dim3(256), 0, stream, (uint32_t*)offsets,
                           (int64_t)E + 1, 0u);
        return check_launch("xma_route_build");
    }
    const int nbits = ceil_log2(E);
    if (n <= kSingleBlockSortIds && E <= kSingleBlockBins) {  // one launch, no workspace
        const size_t lds_one = ((size_t)E * (1024 / kWaveSize) + 1024) * sizeof(uint32_t);
#define XMA_ROUTE_ONE(IdT, OutT)                                                                                     \
    hipLaunchKernelGGL((route_single_block_kernel<IdT, OutT>), dim3(1), dim3(1024), lds_one, stream, (const IdT*)ids, \
                       n, (int)E, nbits, counts, offsets, (OutT*)sorted_ids, (OutT*)perm)
        if (ids_is_i64) {
            if (out_is_i64)
                XMA_ROUTE_ONE(int64_t, int64_t);
            else
                XMA_ROUTE_ONE(int64_t, int32_t);
        } else {
            if (out_is_i64)
                XMA_ROUTE_ONE(int32_t, int64_t);
            else
                XMA_ROUTE_ONE(int32_t, int32_t);
        }
#undef XMA_ROUTE_ONE
        return check_launch("xma_route_build");
    }
    const int64_t units = ceil_div(n, kChunk);
    uint32_t* unit_hist = (uint32_t*)workspace;
    if (units * E <= kFusedScanValues && E <= 256) {  // two launches: histograms, then scan and placement in one
        const size_t hist_lds = (size_t)4 * E * sizeof(uint32_t);
        if (ids_is_i64)
            hipLaunchKernelGGL(block_hist_kernel<int64_t>, dim3((unsigned)units), dim3(256), hist_lds, stream,
                               (const int64_t*)ids, n, (int)E, unit_hist);
        else
            hipLaunchKernelGGL(block_hist_kernel<int32_t>, dim3((unsigned)units), dim3(256), hist_lds, stream,
                               (const int32_t*)ids, n, (int)E, unit_hist);
        const size_t place_lds = ((size_t)6 * E + 4) * sizeof(uint32_t);
#define XMA_SCAN_PLACE(IdT, OutT)                                                                                   \
    hipLaunchKernelGGL((scan_place_kernel<IdT, OutT>), dim3((unsigned)units), dim3(256), place_lds, stream,          \
                       (const IdT*)ids, n, (int)E, nbits, units, (const uint32_t*)unit_hist, counts, offsets,       \
                       (OutT*)sorted_ids, (OutT*)perm)
        if (ids_is_i64) {
            if (out_is_i64)
                XMA_SCAN_PLACE(int64_t, int64_t);
            else
                XMA_SCAN_PLACE(int64_t, int32_t);
        } else {
            if (out_is_i64)
                XMA_SCAN_PLACE(int32_t, int64_t);
            else
                XMA_SCAN_PLACE(int32_t, int32_t);
        }
#undef XMA_SCAN_PLACE
        return check_launch("xma_route_build");
    }
    // four launches: histograms, column scan over the units, scan over the experts, placement; a unit belongs to a
    // block of four waves while four rows of E words fit in LDS, to one wave beyond
    const bool quarters = E <= kQuarterMaxExperts;
    // (measured: 2^17 ids x 1024 experts 8.5 us against 19.2 us for the placement; 2^20 x 256 17.3 against 15.3 us,
    // where a wave that walks 1024 ids writes four adjacent slots per expert)
    const bool place_in_quarters = quarters && E > 256;
    const int wpb = sort_waves_per_block(E);
    const unsigned blocks = (unsigned)ceil_div(units, wpb);
    const size_t lds = (size_t)wpb * E * sizeof(uint32_t);
    const size_t quarter_lds = (size_t)4 * E * sizeof(uint32_t);
    if (quarters) {
        if (ids_is_i64)
            hipLaunchKernelGGL(block_hist_kernel<int64_t>, dim3((unsigned)units), dim3(256), quarter_lds, stream,
                               (const int64_t*)ids, n, (int)E, unit_hist);
        else
            hipLaunchKernelGGL(block_hist_kernel<int32_t>, dim3((unsigned)units), dim3(256), quarter_lds, stream,
                               (const int32_t*)ids, n, (int)E, unit_hist);
    } else if (ids_is_i64) {
        hipLaunchKernelGGL(unit_hist_kernel<int64_t>, dim3(blocks), dim3(wpb * kWaveSize), lds, stream,
                           (const int64_t*)ids, n, (int)E, wpb, unit_hist);
    } else {
        hipLaunchKernelGGL(unit_hist_kernel<int32_t>, dim3(blocks), dim3(wpb * kWaveSize), lds, stream,
                           (const int32_t*)ids, n, (int)E, wpb, unit_hist);
    }
    hipLaunchKernelGGL(unit_scan_kernel, dim3((E + kWaveSize - 1) / kWaveSize), dim3(1024), 0, stream, unit_hist, units,
                       (int)E, counts);
    hipLaunchKernelGGL(offsets_kernel, dim3(1), dim3(1024), 0, stream, (const uint32_t*)counts, (int)E, offsets);
#define XMA_PLACE(IdT, OutT)                                                                                       \
    do {                                                                                                           \
        if (place_in_quarters)                                                                                     \
            hipLaunchKernelGGL((place_quarters_kernel<IdT, OutT>), dim3((unsigned)units), dim3(256), quarter_lds,  \
                               stream, (const IdT*)ids, n, (int)E, nbits, (const uint32_t*)unit_hist,              \
                               (const int32_t*)offsets, (OutT*)sorted_ids, (OutT*)perm);                           \
        else                                                                                                       \
            hipLaunchKernelGGL((place_kernel<IdT, OutT>), dim3(blocks), dim3(wpb * kWaveSize), lds, stream,         \
                               (const IdT*)ids, n, (int)E, nbits, wpb, (const uint32_t*)unit_hist,                 \
                               (const int32_t*)offsets, (OutT*)sorted_ids, (OutT*)perm);                           \
    } while (0)
    if (ids_is_i64) {
        if (out_is_i64)
            XMA_PLACE(int64_t, int64_t);
        else
            XMA_PLACE(int64_t, int32_t);
    } else {
        if (out_is_i64)
            XMA_PLACE(int32_t, int64_t);
        else
            XMA_PLACE(int32_t, int32_t);
    }
#undef XMA_PLACE
    return check_launch("xma_route_build");
}

int xma_route_build(const void* ids, int ids_is_i64, int64_t n, int32_t E, uint32_t* counts, int32_t* offsets,
                    void* sorted_ids, void* perm, int out_is_i64, void* workspace, int64_t workspace_bytes,
                    void* stream_) {
    XMA_REQUIRE(E >= 1 && E <= kMaxExperts, "xma_route_build: num_experts=%d outside [1, %d]", E, kMaxExperts);
    XMA_REQUIRE(n >= 0 && n < ((int64_t)1 << 31), "xma_route_build: n=%lld does not fit int32", (long long)n);
    XMA_REQUIRE(counts && offsets, "xma_route_build: counts/offsets must not be null");
    XMA_REQUIRE(n == 0 || (ids && sorted_ids && perm && workspace), "xma_route_build: null pointer");
    XMA_REQUIRE(workspace_bytes >= xma_route_workspace_bytes(n, E), "xma_route_build: workspace too small (%lld < %lld)",
                (long long)workspace_bytes, (long long)xma_route_workspace_bytes(n, E));
    return route_build_launch(ids, ids_is_i64, n, E, counts, offsets, sorted_ids, perm, out_is_i64, workspace,
                              (hipStream_t)stream_);
}

int xma_offsets_from_sorted(const void* sorted_ids, int ids_is_i64, int64_t n, int32_t E, int32_t* offsets,
                            void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    XMA_REQUIRE(E >= 1 && E <= kMaxExperts, "xma_offsets_from_sorted: num_experts=%d outside [1, %d]", E, kMaxExperts);
    XMA_REQUIRE(n >= 0 && n < ((int64_t)1 << 31), "xma_offsets_from_sorted: n=%lld does not fit int32", (long long)n);
    XMA_REQUIRE(offsets != nullptr && (sorted_ids != nullptr || n == 0), "xma_offsets_from_sorted: null pointer");
    const unsigned blocks = (unsigned)ceil_div(n + 1, 256);
    if (ids_is_i64)
        hipLaunchKernelGGL(offsets_from_sorted_kernel<int64_t>, dim3(blocks), dim3(256), 0, stream,
                           (const int64_t*)sorted_ids, n, (int)E, offsets);
    else
        hipLaunchKernelGGL(offsets_from_sorted_kernel<int32_t>, dim3(blocks), dim3(256), 0, stream,
                           (const int32_t*)sorted_ids, n, (int)E, offsets);
    return check_launch("xma_offsets_from_sorted");
}

int64_t xma_route_build_static_max_bytes(void) { return kStaticScratchWords * (int64_t)sizeof(uint32_t); }

int xma_route_build_static(const void* ids, int ids_is_i64, int64_t n, int32_t E, uint32_t* counts, int32_t* offsets,
                           void* sorted_ids, void* perm, int out_is_i64, void* stream_) {
    XMA_REQUIRE(E >= 1 && E <= kMaxExperts, "xma_route_build_static: num_experts=%d outside [1, %d]", E, kMaxExperts);
    XMA_REQUIRE(n >= 0 && n < ((int64_t)1 << 31), "xma_route_build_static: n=%lld does not fit int32", (long long)n);
    XMA_REQUIRE(counts && offsets, "xma_route_build_static: counts/offsets must not be null");
    XMA_REQUIRE(n == 0 || (ids && sorted_ids && perm), "xma_route_build_static: null pointer");
    const int64_t need = xma_route_workspace_bytes(n, E);
    XMA_REQUIRE(need <= xma_route_build_static_max_bytes(),
                "xma_route_build_static: ceil(n / %d) * num_experts * 4 = %lld bytes of working memory exceed the built-in "
                "%lld; use xma_route_build with a caller-owned workspace",
                kChunk, (long long)need, (long long)xma_route_build_static_max_bytes());
    uint32_t* workspace = static_scratch_for_current_device();
    if (workspace == nullptr) return 2;  // error text already set
    return route_build_launch(ids, ids_is_i64, n, E, counts, offsets, sorted_ids, perm, out_is_i64, workspace,
                              (hipStream_t)stream_);
}

int xma_topk_softmax(const void* logits, int dtype, int64_t T, int32_t E, int32_t k, int64_t ld, void* weights,
                     void* idx, int idx_is_i64, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    XMA_REQUIRE(valid_dtype(dtype), "xma_topk_softmax: bad dtype %d", dtype);
    XMA_REQUIRE(E >= 1 && E <= kMaxExperts, "xma_topk_softmax: E=%d outside [1, %d]", E, kMaxExperts);
    XMA_REQUIRE(k >= 1 && k <= E && k <= kWaveSize, "xma_topk_softmax: k=%d must satisfy 1 <= k <= min(E=%d, 64)", k, E);
    XMA_REQUIRE(T >= 0 && ld >= E, "xma_topk_softmax: bad T=%lld or row stride %lld", (long long)T, (long long)ld);
    if (T == 0) return 0;
    XMA_REQUIRE(logits && weights && idx, "xma_topk_softmax: null pointer");
    // lanes per token: at least k (lane s of a group keeps the s-th selection) and enough for eight experts per lane
    int G = 1;
    while (G < k) G <<= 1;
    while (G < kWaveSize && G * 8 < E) G <<= 1;
    const int per_lane = (int)ceil_div(E, G);
    const int wpb = 4;
    const unsigned blocks = (unsigned)ceil_div(T, (int64_t)wpb * (kWaveSize / G));
#define XMA_TOPK(T_, EPL, IdxT)                                                                                    \
    hipLaunchKernelGGL((topk_softmax_kernel<T_, EPL, IdxT>), dim3(blocks), dim3(wpb * kWaveSize), 0, stream,        \
                       (const T_*)logits, T, (int)E, (int)k, G, ld, (T_*)weights, (IdxT*)idx)
#define XMA_TOPK_E(T_, IdxT)                                                                                       \
    if (E > 512)                                                                                                   \
        hipLaunchKernelGGL((topk_softmax_lds_kernel<T_, IdxT>), dim3((unsigned)T), dim3(kWaveSize),                \
                           (size_t)E * sizeof(uint32_t), stream, (const T_*)logits, T, (int)E, (int)k, ld,         \
                           (T_*)weights, (IdxT*)idx);                                                              \
    else if (per_lane <= 1)                                                                                        \
        XMA_TOPK(T_, 1, IdxT);                                                                                     \
    else if (per_lane <= 2)                                                                                        \
        XMA_TOPK(T_, 2, IdxT);                                                                                     \
    else if (per_lane <= 4)                                                                                        \
        XMA_TOPK(T_, 4, IdxT);                                                                                     \
    else                                                                                                           \
        XMA_TOPK(T_, 8, IdxT)
    XMA_DISPATCH_DTYPE(dtype, T_, if (idx_is_i64) { XMA_TOPK_E(T_, int64_t); } else { XMA_TOPK_E(T_, int32_t); })
#undef XMA_TOPK_E
#undef XMA_TOPK
    return check_launch("xma_topk_softmax");
}

int xma_topk_softmax_bwd(const void* logits, int64_t ld_logits, const void* d_weights, const void* idx,
                         int idx_is_i64, int dtype, int64_t T, int32_t E, int32_t k, void* d_logits, int64_t ld,
                         void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    XMA_REQUIRE(valid_dtype(dtype), "xma_topk_softmax_bwd: bad dtype %d", dtype);
    XMA_REQUIRE(E >= 1 && k >= 1 && k <= E && k <= kWaveSize, "xma_topk_softmax_bwd: bad E=%d / k=%d", E, k);
    XMA_REQUIRE(T >= 0 && ld >= E && ld_logits >= E, "xma_topk_softmax_bwd: bad T or row stride");
    if (T == 0) return 0;
    XMA_REQUIRE(logits && d_weights && idx && d_logits, "xma_topk_softmax_bwd: null pointer");
    int G = 1;  // lanes per token: at least k, and at most eight zero stores per lane
    while (G < k) G <<= 1;
    while (G < kWaveSize && G * 8 < E) G <<= 1;
    const int wpb = 4;
    const unsigned blocks = (unsigned)ceil_div(T, (int64_t)wpb * (kWaveSize / G));
    XMA_DISPATCH_DTYPE(
        dtype, T_,
        if (idx_is_i64) hipLaunchKernelGGL((topk_softmax_bwd_kernel<T_, int64_t>), dim3(blocks), dim3(wpb * kWaveSize),
                                           0, stream, (const T_*)logits, ld_logits, (const T_*)d_weights,
                                           (const int64_t*)idx, T, (int)E, (int)k, G, (T_*)d_logits, ld);
        else hipLaunchKernelGGL((topk_softmax_bwd_kernel<T_, int32_t>), dim3(blocks), dim3(wpb * kWaveSize), 0, stream,
                                (const T_*)logits, ld_logits, (const T_*)d_weights, (const int32_t*)idx, T, (int)E,
                                (int)k, G, (T_*)d_logits, ld))
    return check_launch("xma_topk_softmax_bwd");
}

}  // extern "C"
