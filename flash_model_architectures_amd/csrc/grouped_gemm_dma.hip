// Ragged (per-expert) GEMM for 16-bit element types on gfx950, built around the LDS-DMA load path
// (global_load_lds_dwordx4): tiles travel L2 -> LDS without passing through registers, several
// stages are kept in LDS so that loads stay in flight while a stage is multiplied, and operands whose
// reduction index is strided in HBM are fetched in their HBM layout and transposed by the LDS read
// itself (ds_read_b64_tr_b16).
//
// Tile 256 x 256 per work-group, 4 waves as 2 x 2, one wave per SIMD with the whole 512-register budget:
// each wave owns 128 x 128 (8 x 8 blocks of the 16x16x32 matrix instruction, 256 accumulator registers).  A
// wave that is alone on its SIMD has nobody to hide its stalls, so the main loop is software-pipelined by hand:
// the fragments of the 32-deep reduction block k+1 are read from LDS while block k is multiplied, DMA loads are
// dealt out one every eight matrix instructions, and the order of the three streams is pinned slot by slot.
//
// What bounds the loop (measured): what the L2 has to fetch and deliver.  A compute unit pulls a 256 x 256
// tile's operands from L2 at 128 FLOP per byte, the L2 delivers whole 128-byte lines about 1.5 x faster than
// half lines (so K-contiguous operands are staged 64 reduction elements at a time, 128-byte rows; see
// Ring64x5), and the 32 tiles an XCD runs at a time share their operand panels in its L2 as long as they walk
// the reduction in step (see Kernel::phase).
//
// LDS is a pool of five 32 KiB slabs (all 160 KiB of the compute unit).
// Tile layouts inside a slab:
//   K-contiguous operand (A in TN/NN, W in TN): [256 tile rows][BK k]; the 16-byte chunks of a row are
//     XOR-swizzled by the row number so that the 16 rows a quarter-wave reads in one ds_read_b128 cover all
//     64 banks.
//   K-strided operand (W in NN, both operands in MT): [BK k][256 tile rows], 512 bytes per k row; chunk c
//     of k row r sits at c ^ ((r & 3) << 2), so that the four k rows one transposing read touches fall
//     into different bank groups.
// A DMA load writes lane l's 16 bytes at (wave-uniform LDS base) + 16*l, so the swizzles are applied
// by choosing which HBM chunk each lane fetches.  Masked rows / reduction tails are fetched from a
// 16-byte page of zeros, which keeps every lane active and the outstanding-load count uniform.
#include <type_traits>

#include "grouped_gemm_common.h"

namespace xma {
namespace dma {

constexpr int BM = 256, BN = 256, THREADS = 256, NUM_WAVES = THREADS / 64;
constexpr int WAVES_N = 2, WM = 128, WN = 128, MI = WM / 16, NI = WN / 16;  // 8 x 8 blocks of 16 x 16 per wave
constexpr int OUT_SLABS = 4;  // the epilogue stages the tile through LDS 64 rows (one slab) at a time
constexpr int SLAB_BYTES = 32768;
static_assert(BM == BN, "both operands use the same tile height");

__shared__ __attribute__((aligned(1024))) char slab0[SLAB_BYTES];
__shared__ __attribute__((aligned(1024))) char slab1[SLAB_BYTES];
__shared__ __attribute__((aligned(1024))) char slab2[SLAB_BYTES];
__shared__ __attribute__((aligned(1024))) char slab3[SLAB_BYTES];
__shared__ __attribute__((aligned(1024))) char slab4[SLAB_BYTES];

// The slabs are distinct arrays on purpose: the compiler can then prove that a fragment read of
// one slab does not alias the DMA writes still in flight to the others, and does not drain them.
template <int I>
__device__ __forceinline__ char* slab() {
    static_assert(I >= 0 && I < 5, "slab index");
    if constexpr (I == 0) return slab0;
    if constexpr (I == 1) return slab1;
    if constexpr (I == 2) return slab2;
    if constexpr (I == 3) return slab3;
    return slab4;
}

__device__ __attribute__((aligned(16))) uint32_t g_zero_page[4];  // zero-initialised

typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;
#define XMA_LDS(p) ((__attribute__((address_space(3))) void*)(p))
#define XMA_LDS_S4(p) ((__attribute__((address_space(3))) short4_t*)(p))

__device__ __forceinline__ void compiler_fence() { asm volatile("" ::: "memory"); }

// s_waitcnt with only the vector-memory counter constrained (lgkmcnt = 15, expcnt = 7)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt range");
    compiler_fence();
    __builtin_amdgcn_s_waitcnt((N & 0xF) | (7 << 4) | (0xF << 8) | ((N >> 4) << 14));
    compiler_fence();
}

// s_waitcnt on the vector-memory counter and for every LDS read of this wave (lgkmcnt = 0)
template <int N>
__device__ __forceinline__ void wait_vmcnt_and_lds() {
    static_assert(N >= 0 && N < 64, "vmcnt range");
    compiler_fence();
    __builtin_amdgcn_s_waitcnt((N & 0xF) | (7 << 4) | (0 << 8) | ((N >> 4) << 14));
    compiler_fence();
}

__device__ __forceinline__ void block_barrier() {
    compiler_fence();
    __builtin_amdgcn_s_barrier();
    compiler_fence();
}

// LDS accesses add ONE integer byte offset to a slab, and the variable part of the offset is passed
// through opaque() so that the optimiser cannot split it into a chain of partial sums: the compiler
// attaches the "this access belongs to slab X" information it needs to keep DMA loads to the other
// slabs in flight only to accesses whose address is a short derivation from the array.
__device__ __forceinline__ int opaque(int v) {
    asm("" : "+v"(v));
    return v;
}

// The epilogue requests what it needs from HBM and LDS in batches and uses the values afterwards.  Left alone,
// the compiler sinks each load into the conditional block that uses it and then waits for them one by one;
// pin() makes the value live where it is called, and batch_fence() keeps the scheduler from moving the uses
// up between the requests.
template <typename V>
__device__ __forceinline__ void pin(V& v) {
    asm volatile("" : "+v"(v));
}
__device__ __forceinline__ void batch_fence() { __builtin_amdgcn_sched_barrier(0); }

// ---- tile geometry for a stage depth of BK reduction elements ---------------------------------------
template <int BK>
struct Geometry {
    static constexpr int CPR = BK / 8;            // 16-byte chunks per K-contiguous row
    static constexpr int ROW_BYTES = BK * 2;
    static constexpr int ROWS_PER_LOAD = 64 / CPR;  // tile rows one DMA instruction covers
    static constexpr int LOADS = BK / 2 / NUM_WAVES;  // DMA instructions per wave, operand and stage
    static constexpr int TILE_BYTES = BM * BK * 2;
    static_assert(BK == 32 || BK == 64, "stage depth");

    __device__ static __forceinline__ int swizzle(int row) { return BK == 32 ? (row >> 2) & 3 : (row >> 1) & 7; }

    // K-contiguous tile: byte offset of the fragment (row, reduction elements kb*32 + 8*quarter .. +7)
    __device__ static __forceinline__ int kcontig_offset(int row, int kb, int quarter) {
        return row * ROW_BYTES + (((4 * kb + quarter) ^ swizzle(row)) << 4);
    }
    // K-strided tile: byte offset of the first of the two transposing reads of the fragment
    // (tile rows col0..col0+15, reduction elements kb*32 .. +31).  Within each 16-lane group the
    // instruction hands lane i the i-th 16-bit element of four 16-element rows, where row j is assembled
    // from the 8-byte pieces addressed by lanes 4j..4j+3.  So lane i of group g addresses (k row 8g + i/4,
    // columns 4*(i%4)..+3) and receives four consecutive k of column i; a second read four k rows further
    // down completes the eight reduction elements 8g .. 8g+7 of the MFMA operand.
    __device__ static __forceinline__ int kstrided_offset(int col0, int kb, int lane) {
        const int i = lane & 15, group = lane >> 4;
        const int col = col0 + 4 * (i & 3);
        const int krow0 = kb * 32 + 8 * group + (i >> 2);
        const int chunk = (col >> 3) ^ ((krow0 & 3) << 2);  // (krow0 + 4) & 3 == krow0 & 3
        return krow0 * (BN * 2) + (chunk << 4) + ((col & 4) << 1);
    }
};

template <bool STRIDED>
__device__ __forceinline__ u32x4_t read_fragment(const char* slab_base, int offset) {
    if constexpr (STRIDED) {
        const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(XMA_LDS_S4(slab_base + offset));
        const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(XMA_LDS_S4(slab_base + (offset + 4 * (BN * 2))));
        const u32x2_t a = __builtin_bit_cast(u32x2_t, lo), b = __builtin_bit_cast(u32x2_t, hi);
        return u32x4_t{a.x, a.y, b.x, b.y};
    } else {
        return *reinterpret_cast<const u32x4_t*>(slab_base + offset);
    }
}

// ---- per-thread DMA plan of one operand ---------------------------------------------------------------
// DMA instruction i of wave w fills the 1 KiB block (i * NUM_WAVES + w) of the operand's LDS tile:
//   K-contiguous tile: tile rows [R * (i * NUM_WAVES + w), +R), R = ROWS_PER_LOAD; lane l -> row + l / CPR,
//     physical chunk l % CPR (the logical chunk it fetches is the XOR-swizzled one, and because R * NUM_WAVES
//     is a multiple of the swizzle period it is the same for every i);
//   K-strided tile: k rows {2 * (i * NUM_WAVES + w), +1}; lane l -> k row + l / 32, physical chunk l % 32.
// Three address plans:
//   ROWS     one pointer per instruction (rows that are gathered through an index table or end anywhere),
//   UNIFORM  K-contiguous rows at a constant stride, with one extra jump in the middle of the tile
//            (the up|gate halves of a fused SwiGLU weight tile): one pointer, the rest is scalar arithmetic,
//   STRIDED  K-strided tile: one pointer, constant stride between instructions.
enum LoadPlan { PLAN_ROWS, PLAN_UNIFORM, PLAN_STRIDED };

template <typename T, int BK, LoadPlan PLAN>
struct OperandLoads {
    using G = Geometry<BK>;
    static constexpr int LOADS = G::LOADS;
    static constexpr int RED_STRIDE = PLAN == PLAN_STRIDED ? 2 * NUM_WAVES : 0;  // reduction rows between i and i+1
    const T* ptr[PLAN == PLAN_ROWS ? LOADS : 1];  // HBM address of this lane's chunk in stage 0
    bool valid[PLAN == PLAN_STRIDED ? 1 : LOADS];  // false: always the zero page (row / column outside the operand)
    int64_t load_stride, mid_jump;  // UNIFORM / STRIDED: elements from instruction i to i+1; UNIFORM: extra at LOADS/2
    int64_t step;                   // elements to advance per stage
    int32_t red0;                   // reduction index covered by the lane in stage 0, instruction 0
    int wave_lds;                   // byte offset of the wave's first 1 KiB block inside the operand's LDS tile

    __device__ static __forceinline__ const T* zero_page() { return reinterpret_cast<const T*>(g_zero_page); }

    // ROWS: row_fn(tile row) returns the HBM row base or nullptr.
    template <typename RowFn>
    __device__ __forceinline__ void setup_rows(int wave, int lane, RowFn row_fn) {
        static_assert(PLAN == PLAN_ROWS, "plan");
        const int chunk = (lane % G::CPR) ^ G::swizzle(wave * G::ROWS_PER_LOAD + lane / G::CPR);
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const T* base = row_fn((i * NUM_WAVES + wave) * G::ROWS_PER_LOAD + lane / G::CPR);
            valid[i] = base != nullptr;
            ptr[i] = valid[i] ? base + chunk * 8 : zero_page();
        }
        red0 = chunk * 8;
        step = BK;
        wave_lds = wave * 1024;
    }

    // UNIFORM: tile row r lives at base + r * ld (+ jump for r >= 128); rows_fn(tile row) says whether it exists.
    template <typename ValidFn>
    __device__ __forceinline__ void setup_uniform(int wave, int lane, const T* base, int64_t ld, int64_t jump,
                                                  ValidFn valid_fn) {
        static_assert(PLAN == PLAN_UNIFORM, "plan");
        const int row = wave * G::ROWS_PER_LOAD + lane / G::CPR;
        const int chunk = (lane % G::CPR) ^ G::swizzle(row);
#pragma unroll
        for (int i = 0; i < LOADS; ++i) valid[i] = valid_fn(i * NUM_WAVES * G::ROWS_PER_LOAD + row);
        ptr[0] = base + row * ld + chunk * 8;
        load_stride = NUM_WAVES * G::ROWS_PER_LOAD * ld;
        mid_jump = jump;
        red0 = chunk * 8;
        step = BK;
        wave_lds = wave * 1024;
    }

    // STRIDED: `base` points at (reduction row 0, first tile column); `cols_left` = number of valid columns
    // from there; ld = row stride.
    __device__ __forceinline__ void setup_strided(int wave, int lane, const T* base, int64_t ld, int64_t cols_left) {
        static_assert(PLAN == PLAN_STRIDED, "plan");
        const int krow = wave * 2 + (lane >> 5);
        const int chunk = (lane & 31) ^ ((krow & 3) << 2);  // 2 * NUM_WAVES is a multiple of 4: same for every i
        valid[0] = chunk * 8 < cols_left;
        ptr[0] = valid[0] ? base + (int64_t)krow * ld + chunk * 8 : zero_page();
        load_stride = 2 * NUM_WAVES * ld;
        mid_jump = 0;
        red0 = krow;
        step = (int64_t)BK * ld;
        wave_lds = wave * 1024;
    }

    // Make stage 0 the stage `first` of the reduction (split-K parts start in the middle).
    __device__ __forceinline__ void skip_stages(int64_t first) {
#pragma unroll
        for (int i = 0; i < (PLAN == PLAN_ROWS ? LOADS : 1); ++i) ptr[i] += first * step;
    }

    // Issue this wave's loads I0 <= i < I1 of the stage `stage` into the tile at slab_base + tile_off.
    // MASKED = false is for a stage that lies wholly inside the reduction, of a tile none of whose rows and columns
    // is missing (all_valid): the address is the lane's pointer plus a wave-uniform offset and nothing is compared
    // or selected.  A wave that is alone on its SIMD pays an issue slot for every instruction, and the masked form
    // spends five on each load (a 64-bit compare, a mask and, two selects), the plain one none.
    template <int I0, int I1, bool MASKED>
    __device__ __forceinline__ void issue(char* slab_base, int tile_off, int64_t stage, int64_t red_len) const {
        const int64_t red_left = red_len - stage * BK;  // wave-uniform
        const int64_t stage_off = stage * step;
#pragma unroll
        for (int i = I0; i < I1; ++i) {
            const T* p;
            if constexpr (PLAN == PLAN_ROWS) p = ptr[i] + stage_off;
            else p = ptr[0] + (stage_off + i * load_stride + (i >= LOADS / 2 ? mid_jump : 0));
            if constexpr (MASKED) {
                const bool ok = valid[PLAN == PLAN_STRIDED ? 0 : i] && (red0 + i * RED_STRIDE < red_left);
                // computed for every lane and then selected: a branch around the load would make the number of
                // loads in flight differ between waves
                asm("" : "+v"(p));
                p = ok ? p : zero_page();
            }
            // The wave's share of the LDS address goes through an empty asm that also names the stage, so that the
            // address of every load is ONE scalar add on the spot; left alone, the compiler forms all eighty
            // addresses of a trip round the ring ahead of the loop, runs out of scalar registers and reads them
            // back from vector lanes.  (Not volatile: a volatile asm fences the instruction scheduler, which
            // then cannot spread the loads and LDS reads between the matrix instructions.)
            int w = wave_lds;
            asm("" : "+s"(w) : "s"((int)stage));
            __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t*>(p),
                                             XMA_LDS(slab_base + (tile_off + i * NUM_WAVES * 1024 + w)), 16, 0, 0);
        }
    }

    // true when no row or column of this wave's share of the operand tile is missing
    __device__ __forceinline__ bool all_valid() const {
        bool ok = true;
#pragma unroll
        for (int i = 0; i < (PLAN == PLAN_STRIDED ? 1 : LOADS); ++i) ok = ok && valid[i];
        return ok;
    }
};

// ---- pipeline policies --------------------------------------------------------------------------------------
// A policy says where the tiles of stage j live, which loads the step at cycle position P issues in
// each of its phases (one phase = 32 reduction elements), and how many loads may still be in flight when
// the step reaches its barrier.  Loads are spread evenly over the phases: the texture path of a compute
// unit takes about sixteen cycles per DMA instruction and a wave that issues into a full queue stalls,
// matrix instructions included.
//
// Ring64x5: stage j of 64 reduction elements (two phases of 32) keeps its A tile in slab (2j) % 5 and its B tile
// in slab (2j + 1) % 5, so every DMA instruction of a K-contiguous operand asks for whole 128-byte lines.  At a
// step's barrier the next stage has landed and the A tile of the one after is in flight.  The step's own slabs then
// take the B tile of stage s+2 (during the rest of the step) and the A tile of stage s+3 (during the first phase of
// the next step): every load is issued between one and a half and two and a half phases before the barrier that
// needs it.
struct Ring64x5 {
    static constexpr int BK = 64, CYCLE = 5, KK = 2;
    static constexpr int L = Geometry<BK>::LOADS;
    static constexpr int PHASE_LOADS = L;
    static constexpr int WAIT = L;               // loads that may stay in flight at a step's barrier
    static constexpr int PROLOGUE_WAIT = 2 * L;  // ... and when the first stage is needed
    template <int P> struct At {
        static constexpr int A_SLAB = (2 * P) % 5, A_OFF = 0, B_SLAB = (2 * P + 1) % 5, B_OFF = 0;
    };
    static constexpr int LOOKAHEAD = 2;  // a step at stage s issues loads of stages up to s + LOOKAHEAD
    template <typename K> __device__ static __forceinline__ void prologue(K& k) {
        k.template issue_a<0, 0, L, true>(0); k.template issue_b<0, 0, L, true>(0);
        k.template issue_a<1, 0, L, true>(1); k.template issue_b<1, 0, L, true>(1);
    }
    // load number I (0 <= I < PHASE_LOADS) of phase PH of the step at ring position P on stage s
    template <int P, int PH, int I, bool MASKED, typename K> __device__ static __forceinline__ void issue_one(K& k, int64_t s) {
        if constexpr (PH == 0) k.template issue_a<(P + 2) % CYCLE, I, I + 1, MASKED>(s + 2);
        else k.template issue_b<(P + 2) % CYCLE, I, I + 1, MASKED>(s + 2);
    }
};

template <typename T, int KIND, int EPI, typename Pipe>
struct Kernel {
    static constexpr int BK = Pipe::BK;
    using G = Geometry<BK>;
    static constexpr bool A_STRIDED = KIND == XMA_GEMM_MT;
    static constexpr bool B_STRIDED = KIND != XMA_GEMM_TN;
    static constexpr int BN_OUT = EPI == EPI_PAIRED ? BN / 2 : BN;

    OperandLoads<T, BK, A_STRIDED ? PLAN_STRIDED : PLAN_ROWS> la;
    OperandLoads<T, BK, B_STRIDED ? PLAN_STRIDED : PLAN_UNIFORM> lb;
    int64_t red_len;
    int wave, lane;
    int a_off[4], b_off[4];  // variable parts of the fragment offsets (see fragment_offsets)
    u32x4_t fa[2][MI], fb[2][NI];  // fragments: the 32-deep block being multiplied and the one being read

    template <int P, int I0, int I1, bool MASKED> __device__ __forceinline__ void issue_a(int64_t stage) {
        la.template issue<I0, I1, MASKED>(slab<Pipe::template At<P>::A_SLAB>(), Pipe::template At<P>::A_OFF, stage, red_len);
    }
    template <int P, int I0, int I1, bool MASKED> __device__ __forceinline__ void issue_b(int64_t stage) {
        lb.template issue<I0, I1, MASKED>(slab<Pipe::template At<P>::B_SLAB>(), Pipe::template At<P>::B_OFF, stage, red_len);
    }

    // Byte offsets of this lane's fragments inside an operand tile.  Only the part that is not a
    // compile-time constant goes through opaque(): for the K-contiguous layout the 16-row block adds a
    // constant (the swizzle repeats every 16 rows); for the K-strided layout the 32-deep block adds 16 KiB and
    // the odd 16-column block of a 32-column pair adds 32 bytes (two chunks; the swizzle leaves that bit alone).
    template <bool STRIDED>
    __device__ __forceinline__ void fragment_offsets(int row0, int (&var)[4]) const {
        if constexpr (STRIDED) {
#pragma unroll
            for (int b = 0; b < 4; ++b) var[b] = opaque(G::kstrided_offset(row0 + b * 32, 0, lane));
        } else {
#pragma unroll
            for (int kb = 0; kb < BK / 32; ++kb) var[kb] = opaque(G::kcontig_offset(row0 + (lane & 15), kb, lane >> 4));
        }
    }
    template <bool STRIDED>
    __device__ static __forceinline__ int fragment_offset(const int (&var)[4], int block, int kb) {
        return STRIDED ? var[block >> 1] + (block & 1) * 32 + kb * (32 * BN * 2) : var[kb] + block * (16 * G::ROW_BYTES);
    }
    __device__ __forceinline__ void init_fragments() {
        fragment_offsets<A_STRIDED>((wave / WAVES_N) * WM, a_off);
        fragment_offsets<B_STRIDED>((wave % WAVES_N) * WN, b_off);
    }

    // One fragment of the 32-deep block kb of the stage held at ring position P: A block mi / B block ni.
    template <int P>
    __device__ __forceinline__ u32x4_t read_a(int kb, int mi) const {
        using At = typename Pipe::template At<P>;
        return read_fragment<A_STRIDED>(slab<At::A_SLAB>(), At::A_OFF + fragment_offset<A_STRIDED>(a_off, mi, kb));
    }
    template <int P>
    __device__ __forceinline__ u32x4_t read_b(int kb, int ni) const {
        using At = typename Pipe::template At<P>;
        return read_fragment<B_STRIDED>(slab<At::B_SLAB>(), At::B_OFF + fragment_offset<B_STRIDED>(b_off, ni, kb));
    }
    // All fragments of a block.
    template <int P>
    __device__ __forceinline__ void read_fragments(int kb, u32x4_t (&af)[MI], u32x4_t (&bf)[NI]) const {
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) bf[ni] = read_b<P>(kb, ni);
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) af[mi] = read_a<P>(kb, mi);
    }

    // One phase = one 32-deep block = MI * NI matrix instructions of 16 cycles.  A wave that is alone on its SIMD
    // has nobody to hide its stalls, so the three instruction streams are interleaved by hand: the phase is cut into
    // 32 slots of two matrix instructions (one B block against two A blocks).  Every odd slot also reads one block
    // of the NEXT phase's fragments and every fourth slot issues one DMA load.  The matrix instructions are inline
    // assembly, which the instruction scheduler cannot classify, so the order is pinned with a scheduling fence
    // after each slot.  RP / RKB: ring position and block of the fragments being read; LP / LPH: the step and phase
    // whose loads go out.
    //
    // The granularity and the placement are measured choices (benchmark layer, all launches of a pass, same
    // session): against 16 slots of four instructions with the B blocks read two per slot in the first four slots
    // and the loads in the odd slots, this schedule is 3.3 % faster; with the loads in slot 1 instead of slot 0 of
    // every four 2.6 %; 16 slots with the reads spread out and the loads in even slots 1.4 %.  The kinds differ in
    // the best order of the reads: all A blocks, then all B blocks where both operands cost the same number of LDS
    // instructions (TN, MT), alternating where the transposed operand costs twice as many (NN).  One instruction
    // per slot makes no difference where it compiles (NN: +-0.5 %); for TN and MT the compiler runs out of scalar
    // registers ("illegal VGPR to SGPR copy"), and with the scalar operands of the loads forced through
    // v_readfirstlane it spills thousands of vector registers.
    //
    // The tail tile of an expert's rows runs exactly the same instruction stream on zeros for the rows that do not
    // exist.  Skipping the missing 16-row blocks was measured and is a LOSS: the 32 work-groups an XCD runs at a
    // time share their operand panels through the L2 only while they walk the reduction in step; a tile that
    // finishes early puts its compute unit out of step for the rest of the launch, its requests stop hitting lines
    // its neighbours brought in, and the launch, which is bound by what the L2 has to fetch, gets 13-16 % slower
    // (8 tail tiles among 67 at the benchmark shape).
    template <int RP, int LP, int LPH, bool MASKED>
    __device__ __forceinline__ void phase(int rkb, int cur, int64_t s, f32x4_t (&acc)[MI][NI]) {
        constexpr int SLOTS = 4 * MI;  // 32
        const int nxt = cur ^ 1;
#pragma unroll
        for (int slot = 0; slot < SLOTS; ++slot) {
            const int ni = slot / 4, m0 = (slot & 3) * 2;
            Mma16<T>::run(fb[cur][ni], fa[cur][m0], acc[m0][ni]);
            Mma16<T>::run(fb[cur][ni], fa[cur][m0 + 1], acc[m0 + 1][ni]);
            if (slot % 2 == 1) {
                const int r = slot / 2;  // the r-th of the 16 fragment blocks of the next phase
                if constexpr (KIND == XMA_GEMM_NN) {
                    if (r % 2 == 0) fa[nxt][r / 2] = read_a<RP>(rkb, r / 2);
                    else fb[nxt][r / 2] = read_b<RP>(rkb, r / 2);
                } else {
                    if (r < MI) fa[nxt][r] = read_a<RP>(rkb, r);
                    else fb[nxt][r - MI] = read_b<RP>(rkb, r - MI);
                }
            }
            if (slot % 4 == 0) issue_slot<LP, LPH, MASKED>(slot / 4, s);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    template <int LP, int LPH, bool MASKED>
    __device__ __forceinline__ void issue_slot(int i, int64_t s) {
        // i is a constant after unrolling; the loads of a phase are numbered 0 .. PHASE_LOADS - 1
        switch (i) {
            case 0: Pipe::template issue_one<LP, LPH, 0, MASKED>(*this, s); break;
            case 1: Pipe::template issue_one<LP, LPH, 1, MASKED>(*this, s); break;
            case 2: Pipe::template issue_one<LP, LPH, 2, MASKED>(*this, s); break;
            case 3: Pipe::template issue_one<LP, LPH, 3, MASKED>(*this, s); break;
            case 4: Pipe::template issue_one<LP, LPH, 4, MASKED>(*this, s); break;
            case 5: Pipe::template issue_one<LP, LPH, 5, MASKED>(*this, s); break;
            case 6: Pipe::template issue_one<LP, LPH, 6, MASKED>(*this, s); break;
            default: Pipe::template issue_one<LP, LPH, 7, MASKED>(*this, s); break;
        }
    }
    // One pipeline step at ring position P on stage s.  On entry the fragments of the stage's first block are in
    // registers (set 0).  Phase 0 multiplies block 0 while block 1 is read and the A tile of stage s+2 is requested.
    // Then the step waits until its own LDS reads are done and the loads of stage s+1 have landed, and meets the
    // other waves: stage s+1 is then complete for everybody and nobody reads stage s any more, so its slabs can be
    // refilled while block 1 is multiplied from registers and the first fragments of stage s+1 are read.  A step is
    // branch-free: stages past the end of the reduction fetch the zero page, which keeps the count of loads in
    // flight the same at every step and lets the compiler see that the loop needs no other wait on vector memory.
    template <int P, bool MASKED>
    __device__ __forceinline__ void step(int64_t s, f32x4_t (&acc)[MI][NI]) {
        static_assert(Pipe::KK == 2 && Pipe::PHASE_LOADS == 8, "two phases of eight loads");
        phase<P, P, 0, MASKED>(1, 0, s, acc);
        wait_vmcnt_and_lds<Pipe::WAIT>();
        block_barrier();
        phase<(P + 1) % Pipe::CYCLE, P, 1, MASKED>(0, 1, s, acc);
    }

    template <int P>
    __device__ __forceinline__ void steps_from(int64_t s, int64_t count, f32x4_t (&acc)[MI][NI]) {
        if constexpr (P < Pipe::CYCLE) {
            if (P < count) {
                step<P, true>(s + P, acc);
                steps_from<P + 1>(s, count, acc);
            }
        }
    }
    template <int P, bool MASKED>
    __device__ __forceinline__ void full_cycle(int64_t s, f32x4_t (&acc)[MI][NI]) {
        if constexpr (P < Pipe::CYCLE) {
            step<P, MASKED>(s + P, acc);
            full_cycle<P + 1, MASKED>(s, acc);
        }
    }

    // `plain_steps`: the first that many steps only issue loads of stages that lie wholly inside the reduction, in a
    // tile without missing rows or columns; they take the unmasked form of the loads.
    __device__ __forceinline__ void run_stages(int64_t num_stages, int64_t plain_steps, f32x4_t (&acc)[MI][NI]) {
        read_fragments<0>(0, fa[0], fb[0]);
        int64_t s = 0;
        for (; s + Pipe::CYCLE <= plain_steps; s += Pipe::CYCLE) full_cycle<0, false>(s, acc);
        for (; s + Pipe::CYCLE <= num_stages; s += Pipe::CYCLE) full_cycle<0, true>(s, acc);
        steps_from<0>(s, num_stages - s, acc);  // fewer than CYCLE steps remain
    }

    __device__ __forceinline__ void run(f32x4_t (&acc)[MI][NI]) {
        const int64_t num_stages = (red_len + BK - 1) / BK;
        if (num_stages > 0) {
            Pipe::prologue(*this);
            wait_vmcnt<Pipe::PROLOGUE_WAIT>();
            block_barrier();
            // wave-uniform: validity is a property of rows and columns of the tile, combined over the lanes; the
            // plain and the masked loops issue the same loads and meet at the same barriers, so the waves of a
            // work-group may disagree
            const bool whole = __builtin_amdgcn_readfirstlane(__all((int)(la.all_valid() && lb.all_valid()))) != 0;
            const int64_t plain = whole ? red_len / BK - Pipe::LOOKAHEAD : 0;
            run_stages(num_stages, plain, acc);
            wait_vmcnt<0>();  // the trailing zero-page loads
            // The matrix instructions are inline assembly, so the compiler does not know that the accumulators are
            // still being written when the loop ends and would not keep the distance the hardware needs between a
            // matrix instruction and a read of its result: 32 idle cycles cover it.
            asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
        }
        block_barrier();  // every wave is done reading the slabs; no load is in flight any more
    }
};

template <typename T, int KIND, int EPI, typename Pipe>
__global__ __launch_bounds__(THREADS) void grouped_gemm_dma_kernel(const GemmParams P) {
    using K = Kernel<T, KIND, EPI, Pipe>;
    constexpr int PV = 8;
    constexpr int BN_OUT = K::BN_OUT;

    const int tid = threadIdx.x;
    K k;
    k.lane = tid & 63;
    k.wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    int row_tile, col_tile;
    TileWork work;
    work.parts = 1;
    if constexpr (KIND == XMA_GEMM_MT) {
        if (!locate_tile<true>(P.row_tiles_max * P.num_experts, P.col_tiles, row_tile, col_tile)) return;
    } else {
        if (!locate_work(P.tile_count[0], P.col_tiles, P.num_cu, (P.k + K::BK - 1) / K::BK, work)) return;
        row_tile = work.row_tile;
        col_tile = work.col_tile;
    }

    const T* A = reinterpret_cast<const T*>(P.a);
    const T* B = reinterpret_cast<const T*>(P.b);

    int expert;
    int64_t m_begin, m_end, tile_i0 = 0, n0;
    if constexpr (KIND == XMA_GEMM_MT) {
        const int slot = row_tile / P.row_tiles_max;
        tile_i0 = (int64_t)(row_tile % P.row_tiles_max) * BM;
        if (P.expert_order != nullptr) {  // experts in descending order of their row counts
            const int32_t* record = P.expert_order + 4 * slot;
            expert = record[0];
            m_begin = record[1];
            m_end = record[2];
        } else {
            expert = slot;
            m_begin = P.offsets[expert];
            m_end = P.offsets[expert + 1];
        }
        k.red_len = m_end - m_begin;
        n0 = (int64_t)col_tile * BN;
    } else {
        expert = P.tile_expert[row_tile];
        m_begin = P.tile_row0[row_tile];
        const int64_t e_end = P.offsets[expert + 1];
        m_end = m_begin + BM < e_end ? m_begin + BM : e_end;
        k.red_len = P.k;
        n0 = (int64_t)col_tile * BN_OUT;
    }

    // ---- operand load plans ----
    if constexpr (KIND == XMA_GEMM_MT) {
        k.la.setup_strided(k.wave, k.lane, A + m_begin * P.lda + tile_i0, P.lda, P.n - tile_i0);
        k.lb.setup_strided(k.wave, k.lane, B + m_begin * P.ldb + n0, P.ldb, P.k - n0);
    } else {
        // The three ways of finding a row's source are told apart once, outside the per-row code, and rows past
        // the end look up the tile's first row (which always exists) and are then dropped: with a branch per
        // row the eight index loads of a lane would wait for each other.
        auto plan_rows = [&](auto source_of) {
            k.la.setup_rows(k.wave, k.lane, [&](int r) -> const T* {
                const int64_t p = m_begin + r;
                const bool exists = p < m_end;
                const T* row = A + source_of(exists ? p : m_begin) * P.lda;
                return exists ? row : nullptr;
            });
        };
        const uint32_t fan_out = (uint32_t)P.in_fan_out;
        if (P.in_index == nullptr)
            plan_rows([&](int64_t p) { return p; });
        else if (P.idx_is_i64)
            plan_rows([&](int64_t p) {
                return (int64_t)((uint32_t)reinterpret_cast<const int64_t*>(P.in_index)[p] / fan_out);
            });
        else
            plan_rows([&](int64_t p) {
                return (int64_t)((uint32_t)reinterpret_cast<const int32_t*>(P.in_index)[p] / fan_out);
            });
        const T* W = B + (int64_t)expert * P.b_expert_stride;
        if constexpr (KIND == XMA_GEMM_TN) {
            if constexpr (EPI == EPI_PAIRED) {
                // tile rows 0..127: weight rows n0 + r (up half); rows 128..255: P.n / 2 + n0 + r - 128 (gate half)
                const int64_t half = P.n / 2;
                k.lb.setup_uniform(k.wave, k.lane, W + n0 * P.ldb, P.ldb, (half - BN_OUT) * P.ldb,
                                   [&](int r) { return n0 + (r % BN_OUT) < half; });
            } else {
                k.lb.setup_uniform(k.wave, k.lane, W + n0 * P.ldb, P.ldb, 0, [&](int r) { return n0 + r < P.n; });
            }
        } else {
            k.lb.setup_strided(k.wave, k.lane, W + n0, P.ldb, P.n - n0);
        }
    }
    if constexpr (KIND != XMA_GEMM_MT) {
        if (work.parts > 1) {
            const int64_t stages = (k.red_len + K::BK - 1) / K::BK;
            const int64_t first = work.part * stages / work.parts, end = (work.part + 1) * stages / work.parts;
            k.la.skip_stages(first);
            k.lb.skip_stages(first);
            k.red_len = (end * K::BK < k.red_len ? end * K::BK : k.red_len) - first * K::BK;
        }
    }
    k.init_fragments();
    f32x4_t acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

    k.run(acc);

    // ---- split-K: every part parks its accumulators; the part that arrives last adds them up in part order
    // (so the result does not depend on the arrival order) and goes on to the epilogue ----
    if constexpr (KIND != XMA_GEMM_MT) {
        if (work.parts > 1) {
            // The parts of a tile run on different XCDs, whose L2 caches are not kept coherent with each other.  Fences
            // at device scope would do (each writes back and invalidates the XCD's whole L2, once per wave, under
            // every other work-group of the XCD: 150-200 k cycles per exchange, measured).  Instead the partial sums
            // and the arrival counter are accessed with relaxed DEVICE-SCOPE ATOMIC stores, loads and one
            // read-modify-write.  What the exchange relies on, and where each piece comes from:
            //   (1) a device-scope atomic access is performed at the level of the memory hierarchy that all XCDs
            //       share, never out of an XCD's private L2: the gfx942/gfx950 memory model of the compiler gives such
            //       accesses the sc1 bit for exactly that reason (atomicity across the XCDs of one device);
            //   (2) `s_waitcnt vmcnt(0)` returns when every earlier vector-memory access of the wave, stores
            //       included, has been acknowledged by the level that performs it;
            //   (3) the work-group barrier (with its release / acquire fences at work-group scope, which also stop
            //       the compiler from moving memory accesses across it) orders the four waves: when thread 0 counts
            //       the arrival, all partial sums of the work-group have been performed;
            //   (4) the read-modify-write on the counter is performed at the same shared level, so the part that
            //       reads parts - 1 comes after every other part's sums; its loads, device-scope atomics again, are
            //       issued after a further work-group barrier and cannot be satisfied from a stale line of its L2.
            // The compiler cannot reorder any of this: the waits carry memory clobbers, the barriers are fences, and
            // atomics are never merged, widened or hoisted across them.
            auto part_buffer = [&](int part) {
                return reinterpret_cast<uint64_t*>(P.split_partials +
                                                   (int64_t)(part * work.split_tiles + work.split_tile) * kSplitTileFloats);
            };
            uint64_t* mine = part_buffer(work.part);
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                    for (int g = 0; g < 2; ++g) {
                        const float2 v{acc[mi][ni][2 * g], acc[mi][ni][2 * g + 1]};
                        __hip_atomic_store(mine + ((mi * NI + ni) * 2 + g) * THREADS + tid, __builtin_bit_cast(uint64_t, v),
                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
            wait_vmcnt<0>();  // this wave's partial sums have reached memory ...
            __syncthreads();  // ... and so have everybody else's, before the arrival is counted
            int* arrivals = reinterpret_cast<int*>(slab<0>());
            if (tid == 0)
                arrivals[0] = __hip_atomic_fetch_add(P.split_counters + work.split_tile, 1, __ATOMIC_RELAXED,
                                                     __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            const bool last = arrivals[0] == work.parts - 1;
            __syncthreads();  // the slab is reused below
            if (!last) return;
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
            // The sums are requested 32 loads at a time and added afterwards: with all 256 accumulators live the
            // compiler otherwise fetches them one by one, a full memory latency each.
            for (int part = 0; part < work.parts; ++part) {
                const uint64_t* src = part_buffer(part);
#pragma unroll
                for (int m2 = 0; m2 < MI / 2; ++m2) {
                    uint64_t v[2][NI][2];
#pragma unroll
                    for (int h = 0; h < 2; ++h)
#pragma unroll
                        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                            for (int g = 0; g < 2; ++g)
                                v[h][ni][g] = __hip_atomic_load(src + (((2 * m2 + h) * NI + ni) * 2 + g) * THREADS + tid,
                                                                __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    batch_fence();
#pragma unroll
                    for (int h = 0; h < 2; ++h)
#pragma unroll
                        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                            for (int g = 0; g < 2; ++g) pin(v[h][ni][g]);
#pragma unroll
                    for (int h = 0; h < 2; ++h)
#pragma unroll
                        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                            for (int g = 0; g < 2; ++g) {
                                const float2 f = __builtin_bit_cast(float2, v[h][ni][g]);
                                acc[2 * m2 + h][ni][2 * g] += f.x;
                                acc[2 * m2 + h][ni][2 * g + 1] += f.y;
                            }
                    batch_fence();
                }
            }
        }
    }

    // ---- epilogue: accumulators -> LDS (slab mi holds the 64 tile rows {wr*128 + mi*32 + 0..31}) -> HBM ----
    // Store phase: each thread owns one 16-byte chunk column (cc) and, per slab, the IT buffer rows
    // tid / 32 + 8 * it.  What the rows need from HBM (scatter indices, the saved pre-activation of the
    // activation backward) is requested in batches before it is used: the indices of all four slabs before the
    // accumulators are packed (and waited for after that), a slab's pre-activations one slab ahead.
    T* C = reinterpret_cast<T*>(P.c);
    constexpr int C_CHUNKS = BN / PV;             // 32
    constexpr int ROW_STEP = THREADS / C_CHUNKS;  // 8
    constexpr int IT = 64 / ROW_STEP;             // 8
    // Per-lane coordinates are derived from a fresh, opaque copy of the thread index: derived from `tid` they
    // would be the values computed before the main loop, which the compiler then keeps in scratch memory
    // across the loop and reloads in the middle of the epilogue's batched requests.
    // A wave that is alone on its SIMD issues one vector instruction every 4-5 cycles, so this part of the kernel
    // is bound by its instruction count: row arithmetic is 32-bit and relative to the tile (the thread's first
    // buffer row r0 plus a compile-time constant), and whether a row exists is one compare against a scalar where
    // the row is used, not a mark kept per row.
    const int etid = opaque(tid);
    const int cc = etid & (C_CHUNKS - 1);
    const int r0 = (etid / C_CHUNKS) & (ROW_STEP - 1);
    auto buffer_row = [&](int it) { return r0 + it * ROW_STEP; };
    // tile row of buffer row r0 + 8 * it of slab mi, less r0: buffer rows 0..31 are tile rows mi*32 + 0..31, buffer
    // rows 32..63 the same rows of the lower wave row (+128)
    auto row_base = [](int mi, int it) { return (it >> 2) * 128 + mi * 32 + (it & 3) * ROW_STEP; };
    const int rows_here = (int)(m_end - m_begin);  // 1..256
    auto row_exists = [&](int mi, int it) { return r0 < rows_here - row_base(mi, it); };
    // a row of the tile that exists: the wanted one or, past the end, the last one
    auto safe_row = [&](int mi, int it) {
        const int r = r0 + row_base(mi, it);
        return (uint32_t)(r < rows_here ? r : rows_here - 1);
    };

    int32_t orow[OUT_SLABS][IT];  // output row of each owned row (of the last existing row for rows past the end)
    if constexpr (KIND != XMA_GEMM_MT) {
        auto fill = [&](auto index_of) {
#pragma unroll
            for (int mi = 0; mi < OUT_SLABS; ++mi)
#pragma unroll
                for (int it = 0; it < IT; ++it) orow[mi][it] = index_of(safe_row(mi, it));
            batch_fence();  // the loads stay in flight while the accumulators are packed; they are waited for after that
        };
        if (EPI == EPI_BACKWARD || P.out_index == nullptr) {  // that epilogue only writes grouped rows
            const int32_t first = (int32_t)m_begin;
            fill([&](uint32_t r) { return first + (int32_t)r; });
        } else if (P.idx_is_i64) {
            const int64_t* index = reinterpret_cast<const int64_t*>(P.out_index) + m_begin;
            fill([&](uint32_t r) { return (int32_t)index[r]; });
        } else {
            const int32_t* index = reinterpret_cast<const int32_t*>(P.out_index) + m_begin;
            fill([&](uint32_t r) { return index[r]; });
        }
    }

    // Activation backward: the saved pre-activation chunks (the two halves of a gated one; tanh-GELU has a single
    // half, fetched twice) of the rows of slab mi, double-buffered so that slab mi+1 is on its way from HBM while
    // slab mi is processed
    constexpr bool SWBWD = EPI == EPI_BACKWARD;
    u32x4_t hu[SWBWD ? 2 : 1][IT], hg[SWBWD ? 2 : 1][IT];
    auto load_saved = [&](int mi, u32x4_t (&up)[IT], u32x4_t (&gate)[IT]) {
        // branch-free: rows / columns outside the tile's part of the operand re-read a valid chunk
        const int64_t n = n0 + cc * PV < P.n ? n0 + cc * PV : 0;
        const int64_t second_half = P.act == ACT_GELU_TANH ? 0 : P.n;
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const T* h = reinterpret_cast<const T*>(P.aux) + (m_begin + safe_row(mi, it)) * P.ld_aux;
            up[it] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(h + n));
            gate[it] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(h + second_half + n));
        }
    };
    if constexpr (SWBWD) load_saved(0, hu[0], hg[0]);

    // MFMA result register r of lane l in block (mi, ni): tile row 16*mi + l%16, tile column 16*ni + 4*(l/16) + r.
    // Slab s holds the tile rows {wr*128 + s*32 + 0..31} of both wave rows as buffer rows wr*32 + 0..31, i.e. the
    // blocks mi = 2s and 2s+1.  A 512-byte LDS row holds 32 chunks of 8 columns; chunk c of buffer row br sits at
    // c ^ (br & 31).
    {
        const int wn0 = (k.wave % WAVES_N) * WN;
        const int br0 = (k.wave / WAVES_N) * 32 + (etid & 15);  // buffer row of the even block of a slab
        const int quarter = (etid >> 4) & 3;
        // Forward kinds: the expert's bias row, added to the fp32 sums before they are rounded.  Tile column c is
        // weight row n0 + c, or for a gated tile n0 + c (c < 128) and N/2 + n0 + c - 128 (c >= 128).
        float bias[KIND == XMA_GEMM_TN ? NI : 1][KIND == XMA_GEMM_TN ? 4 : 1];
        bool with_bias = false;
        if constexpr (KIND == XMA_GEMM_TN) {
            with_bias = P.bias != nullptr;
            if (with_bias) {
                const T* row = reinterpret_cast<const T*>(P.bias) + (int64_t)expert * P.ld_bias;
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) {
                    const int c = wn0 + ni * 16 + 4 * quarter;
                    int64_t n;
                    bool exists;
                    if constexpr (EPI == EPI_PAIRED) {
                        const int64_t half_n = P.n / 2;
                        n = n0 + (c % BN_OUT) + (c >= BN_OUT ? half_n : 0);
                        exists = n0 + (c % BN_OUT) < half_n;
                    } else {
                        n = n0 + c;
                        exists = n < P.n;
                    }
                    const uint2 raw = *reinterpret_cast<const uint2*>(row + (exists ? n : 0));
                    float v[8];
                    Elem<T>::unpack(make_uint4(raw.x, raw.y, 0u, 0u), v);
#pragma unroll
                    for (int q = 0; q < 4; ++q) bias[ni][q] = exists ? v[q] : 0.0f;
                }
            }
        }
        // (the bias is a copy of the code of its own: a wave alone on its SIMD pays for every instruction, and as
        // one copy the compiler adds a selected zero to every sum of a launch that has no bias)
        auto write_rows = [&](char* buf, const f32x4_t (&even)[NI], const f32x4_t (&odd)[NI], auto bias_tag) {
            constexpr bool BIAS = decltype(bias_tag)::value;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int br = br0 + 16 * h;
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) {
                    const f32x4_t& a = h == 0 ? even[ni] : odd[ni];
                    const int c = wn0 + ni * 16 + 4 * quarter;
                    const int chunk = (c >> 3) ^ (br & 31);
                    float v[4] = {a[0], a[1], a[2], a[3]};
                    if constexpr (BIAS) {
#pragma unroll
                        for (int q = 0; q < 4; ++q) v[q] += bias[KIND == XMA_GEMM_TN ? ni : 0][KIND == XMA_GEMM_TN ? q : 0];
                    }
                    *reinterpret_cast<uint2*>(buf + br * (BN * 2) + (chunk << 4) + (quarter & 1) * 8) =
                        make_uint2(Elem<T>::pack2(v[0], v[1]), Elem<T>::pack2(v[2], v[3]));
                }
            }
        };
        auto write_all = [&](auto bias_tag) {
            write_rows(slab<0>(), acc[0], acc[1], bias_tag);
            write_rows(slab<1>(), acc[2], acc[3], bias_tag);
            write_rows(slab<2>(), acc[4], acc[5], bias_tag);
            write_rows(slab<3>(), acc[6], acc[7], bias_tag);
        };
        if (KIND == XMA_GEMM_TN && with_bias) write_all(std::true_type{});
        else write_all(std::false_type{});
    }
    if constexpr (KIND != XMA_GEMM_MT) {
        batch_fence();
#pragma unroll
        for (int mi = 0; mi < OUT_SLABS; ++mi)
#pragma unroll
            for (int it = 0; it < IT; ++it) pin(orow[mi][it]);
    }
    __syncthreads();

    auto store_rows = [&](const char* buf, auto mi_tag, const int32_t (&out_row)[IT]) {
        constexpr int mi = decltype(mi_tag)::value;
        auto chunk_at = [&](int br, int c) {
            return *reinterpret_cast<const u32x4_t*>(buf + br * (BN * 2) + ((c ^ (br & 31)) << 4));
        };
        auto to_uint4 = [](const u32x4_t& v) { return make_uint4(v[0], v[1], v[2], v[3]); };
        // the thread's chunk of each of its IT rows of the slab, requested together
        auto read_own_chunks = [&](u32x4_t (&v)[IT]) {
#pragma unroll
            for (int it = 0; it < IT; ++it) v[it] = chunk_at(buffer_row(it), cc);
            batch_fence();
#pragma unroll
            for (int it = 0; it < IT; ++it) pin(v[it]);
        };
        if constexpr (KIND == XMA_GEMM_MT) {
            const int64_t j = n0 + cc * PV;
            T* out = C + (int64_t)expert * P.c_expert_stride + j;
            u32x4_t v[IT];
            read_own_chunks(v);
#pragma unroll
            for (int it = 0; it < IT; ++it) {
                const int64_t i = tile_i0 + r0 + row_base(mi, it);
                // streaming store: a weight gradient is read again only by the optimizer, so it should not push the
                // operand panels of the running tiles out of the caches (1-2 % on this kind)
                if (i < P.n && j < P.k) __builtin_nontemporal_store(v[it], reinterpret_cast<u32x4_t*>(out + i * P.ldc));
            }
        } else if constexpr (EPI == EPI_PLAIN) {
            const int64_t n = n0 + cc * PV;
            u32x4_t v[IT];
            read_own_chunks(v);
            if (KIND == XMA_GEMM_TN && P.act == ACT_GELU_TANH) {
                // tanh-GELU of the product; the rounded product itself is kept as the pre-activation
#pragma unroll
                for (int it = 0; it < IT; ++it) {
                    if (!row_exists(mi, it) || n >= P.n) continue;
                    const int64_t p = m_begin + r0 + row_base(mi, it);
                    if (P.aux) *reinterpret_cast<u32x4_t*>(reinterpret_cast<T*>(P.aux) + p * P.ld_aux + n) = v[it];
                    float h[PV], o[PV];
                    Elem<T>::unpack(to_uint4(v[it]), h);
#pragma unroll
                    for (int q = 0; q < PV; ++q) o[q] = gelu_tanh_forward<true>(h[q]);
                    *reinterpret_cast<uint4*>(C + (int64_t)out_row[it] * P.ldc + n) = Elem<T>::pack(o);
                }
            } else {
#pragma unroll
                for (int it = 0; it < IT; ++it)
                    if (row_exists(mi, it) && n < P.n)
                        __builtin_nontemporal_store(v[it], reinterpret_cast<u32x4_t*>(C + (int64_t)out_row[it] * P.ldc + n));
            }
        } else if constexpr (EPI == EPI_PAIRED) {
            // The slab row holds 16 chunks of the up half, then the 16 matching chunks of the gate half.  Thread
            // cc handles chunk pair cc % 16 on every other owned row (even `it` for cc < 16, odd otherwise), so
            // that every lane computes.
            constexpr int HALF_CHUNKS = C_CHUNKS / 2;
            const int64_t half_n = P.n / 2;
            const int pair = cc % HALF_CHUNKS;
            const int64_t j = n0 + pair * PV;
            const bool odd = cc >= HALF_CHUNKS;
            const int r1 = r0 + (odd ? ROW_STEP : 0);  // the thread's first buffer row among those it computes
            u32x4_t ups[IT / 2], gates[IT / 2];
#pragma unroll
            for (int it2 = 0; it2 < IT / 2; ++it2) {
                const int br = r1 + 2 * it2 * ROW_STEP;
                ups[it2] = chunk_at(br, pair);
                gates[it2] = chunk_at(br, pair + HALF_CHUNKS);
            }
            batch_fence();
#pragma unroll
            for (int it2 = 0; it2 < IT / 2; ++it2) {
                pin(ups[it2]);
                pin(gates[it2]);
            }
            // one copy of the loop per activation, chosen once: inside it the activation is a constant
            auto rows = [&](auto act_tag) {
                constexpr int ACT = decltype(act_tag)::value;
#pragma unroll
                for (int it2 = 0; it2 < IT / 2; ++it2) {
                    const int32_t row_out = odd ? out_row[2 * it2 + 1] : out_row[2 * it2];
                    if (r1 >= rows_here - row_base(mi, 2 * it2) || j >= half_n) continue;
                    const int64_t p = m_begin + r1 + row_base(mi, 2 * it2);
                    const u32x4_t up = ups[it2], gate = gates[it2];
                    if (P.aux) {
                        T* h = reinterpret_cast<T*>(P.aux) + p * P.ld_aux;
                        __builtin_nontemporal_store(up, reinterpret_cast<u32x4_t*>(h + j));
                        __builtin_nontemporal_store(gate, reinterpret_cast<u32x4_t*>(h + half_n + j));
                    }
                    float u[PV], g[PV], o[PV];
                    Elem<T>::unpack(to_uint4(up), u);
                    Elem<T>::unpack(to_uint4(gate), g);
#pragma unroll
                    for (int q = 0; q < PV; ++q) o[q] = gated_forward<true>(ACT, u[q], g[q]);
                    { const uint4 pk = Elem<T>::pack(o); __builtin_nontemporal_store(u32x4_t{pk.x, pk.y, pk.z, pk.w}, reinterpret_cast<u32x4_t*>(C + (int64_t)row_out * P.ldc + j)); }
                }
            };
            if (P.act == ACT_SWIGLU) rows(std::integral_constant<int, ACT_SWIGLU>{});
            else rows(std::integral_constant<int, ACT_GLU>{});
        } else {  // EPI_BACKWARD
            const int64_t n = n0 + cc * PV;
            if constexpr (mi + 1 < OUT_SLABS) load_saved(mi + 1, hu[(mi + 1) & 1], hg[(mi + 1) & 1]);
            u32x4_t dv[IT];
            read_own_chunks(dv);
            auto rows = [&](auto act_tag) {
                constexpr int ACT = decltype(act_tag)::value;
#pragma unroll
                for (int it = 0; it < IT; ++it) {
                    if (!row_exists(mi, it) || n >= P.n) continue;
                    float u[PV], g[PV], d[PV], du[PV], dg[PV];
                    Elem<T>::unpack(to_uint4(hu[mi & 1][it]), u);
                    Elem<T>::unpack(to_uint4(hg[mi & 1][it]), g);
                    Elem<T>::unpack(to_uint4(dv[it]), d);
                    T* out = C + (int64_t)out_row[it] * P.ldc;
                    if constexpr (ACT == ACT_GELU_TANH) {
#pragma unroll
                        for (int q = 0; q < PV; ++q) du[q] = gelu_tanh_backward<true>(u[q], d[q]);
                        *reinterpret_cast<uint4*>(out + n) = Elem<T>::pack(du);
                    } else {
#pragma unroll
                        for (int q = 0; q < PV; ++q) gated_backward<true>(ACT, u[q], g[q], d[q], du[q], dg[q]);
                        { const uint4 a = Elem<T>::pack(du), b = Elem<T>::pack(dg); __builtin_nontemporal_store(u32x4_t{a.x, a.y, a.z, a.w}, reinterpret_cast<u32x4_t*>(out + n)); __builtin_nontemporal_store(u32x4_t{b.x, b.y, b.z, b.w}, reinterpret_cast<u32x4_t*>(out + P.n + n)); }
                    }
                }
            };
            if (P.act == ACT_SWIGLU) rows(std::integral_constant<int, ACT_SWIGLU>{});
            else if (P.act == ACT_GLU) rows(std::integral_constant<int, ACT_GLU>{});
            else rows(std::integral_constant<int, ACT_GELU_TANH>{});
        }
    };
    store_rows(slab<0>(), std::integral_constant<int, 0>{}, orow[0]);
    store_rows(slab<1>(), std::integral_constant<int, 1>{}, orow[1]);
    store_rows(slab<2>(), std::integral_constant<int, 2>{}, orow[2]);
    store_rows(slab<3>(), std::integral_constant<int, 3>{}, orow[3]);
}

// Compute units of the current device, rounded down to a multiple of the XCD count and capped at the
// number of split slots (the split-K scheme treats that many tiles as one round).
static int compute_units() {
    // asked of the calling thread's current device on every launch (a host-side attribute lookup)
    int device = 0, count = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || count < kNumXcd)
        count = kSplitSlots;
    count = count > kSplitSlots ? kSplitSlots : count;
    return count / kNumXcd * kNumXcd;
}

template <typename T, int KIND, int EPI, typename Pipe>
static int launch(const xma_grouped_gemm_args& a, hipStream_t stream) {
    GemmParams P;
    fill_params(a, P);
    int64_t grid;
    if (KIND == XMA_GEMM_MT) {
        P.row_tiles_max = (int32_t)ceil_div(a.n, BM);
        P.col_tiles = (int32_t)ceil_div(a.k, BN);
        grid = grid_for_tiles((int64_t)P.row_tiles_max * a.num_experts, P.col_tiles);
        if (a.workspace != nullptr) {  // size checked by the caller
            int32_t* records = reinterpret_cast<int32_t*>(a.workspace);
            hipLaunchKernelGGL(build_expert_order_kernel, dim3(1), dim3(1024), 0, stream, a.expert_offsets,
                               a.num_experts, records);
            P.expert_order = records;
        }
    } else {
        const int64_t rt = max_row_tiles(a.rows, a.num_experts, BM);
        int32_t* ws = reinterpret_cast<int32_t*>(a.workspace);
        P.tile_count = ws;
        P.tile_expert = ws + 4;
        P.tile_row0 = ws + 4 + rt;
        P.row_tiles_max = (int32_t)rt;
        // the split-K region is the tail of the workspace
        char* split = reinterpret_cast<char*>(a.workspace) +
                      (xma_grouped_gemm_workspace_bytes(a.num_experts, a.rows) - split_region_bytes());
        P.split_counters = reinterpret_cast<int32_t*>(split);
        P.split_partials = reinterpret_cast<float*>(split + kSplitSlots * sizeof(int32_t));
        P.num_cu = compute_units();
        const int bn_out = EPI == EPI_PAIRED ? BN / 2 : BN;
        const int64_t n_out = EPI == EPI_PAIRED ? a.n / 2 : a.n;
        P.col_tiles = (int32_t)ceil_div(n_out, bn_out);
        grid = grid_for_work(rt * P.col_tiles);
        hipLaunchKernelGGL(build_row_tiles_kernel, dim3(1), dim3(1024), 0, stream, a.expert_offsets, a.num_experts, BM,
                           ws + 4, ws + 4 + rt, ws, P.split_counters);
    }
    XMA_REQUIRE(grid < ((int64_t)1 << 31), "xma_grouped_gemm: %lld tiles exceed the grid limit", (long long)grid);
    hipLaunchKernelGGL((grouped_gemm_dma_kernel<T, KIND, EPI, Pipe>), dim3((unsigned)grid), dim3(THREADS), 0, stream, P);
    return check_launch("xma_grouped_gemm");
}

template <typename T>
static int dispatch(const xma_grouped_gemm_args& a, hipStream_t stream) {
    using PipeTN = Ring64x5;
    using PipeNN = Ring64x5;
    using PipeMT = Ring64x5;
    int shape = EPI_PLAIN, act = ACT_NONE;
    split_epilogue(a.epilogue, shape, act);
    switch (a.kind) {
        case XMA_GEMM_TN:
            if (shape == EPI_PAIRED) return launch<T, XMA_GEMM_TN, EPI_PAIRED, PipeTN>(a, stream);
            return launch<T, XMA_GEMM_TN, EPI_PLAIN, PipeTN>(a, stream);
        case XMA_GEMM_NN:
            if (shape == EPI_BACKWARD) return launch<T, XMA_GEMM_NN, EPI_BACKWARD, PipeNN>(a, stream);
            return launch<T, XMA_GEMM_NN, EPI_PLAIN, PipeNN>(a, stream);
        default:
            return launch<T, XMA_GEMM_MT, EPI_PLAIN, PipeMT>(a, stream);
    }
}

}  // namespace dma

// 16-bit element types; the weight-gradient layout only without a fused row gather (its reduction rows
// would need an index lookup per stage).
bool dma_gemm_supports(const xma_grouped_gemm_args& a) {
    if (a.dtype != XMA_BF16 && a.dtype != XMA_F16) return false;
    if (a.kind == XMA_GEMM_MT && a.in_index != nullptr) return false;
    return true;
}

int launch_dma_gemm(const xma_grouped_gemm_args& a, hipStream_t stream) {
    return a.dtype == XMA_BF16 ? dma::dispatch<bf16_t>(a, stream) : dma::dispatch<f16_t>(a, stream);
}

}  // namespace xma
