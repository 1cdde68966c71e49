// Guarded bf16 GEMM for gfx950: C[M,N] = A[M,K] * B[K,N], row-major, fp32
// accumulation in ascending k, bf16 (round-to-nearest-even) output.
//
// MFMA-bound: 2*M*N*K flop. One work-group of 512 threads (8 wavefronts) owns one
// 256x256 tile of C and walks K in steps of 64 through two LDS buffers:
//   global -> LDS       buffer_load ... lds: every wave-wide load moves 64 x 16 bytes straight
//                       into 1 KiB of LDS, no registers and no LDS store instructions in
//                       between. Lane l of a load fills the l-th 16-byte slot of that KiB and
//                       is free in what it fetches, so the tiles are kept unpadded and
//                       XOR-swizzled: the slot a piece lands in is its natural slot XOR a few
//                       bits of its row, chosen so that every fragment read below touches
//                       each LDS bank once.
//                       A tile: [256 rows][64 k], two rows to a 256-byte line of sixteen
//                       slots, slot = ((row & 1) * 8 + k / 8) ^ (line & 15).
//                       B tile: as it sits in memory, [64 k][256 cols], eight 64-byte granules
//                       to a row, granule = (col / 32) ^ ((k & 3) | ((k >> 1) & 4)).
//   LDS -> MFMA         v_mfma_f32_32x32x16_bf16; wave (wm, wn) of the 2x4 wave grid
//                       accumulates a 128x64 sub-tile = 4x2 blocks of 32x32
// An MFMA operand wants eight consecutive k per lane. A has them contiguous in memory; for B
// (k is the strided dimension) the transposing LDS read of gfx950, ds_read_b64_tr_b16, turns
// four rows of four columns into four k of one column per lane, two of them per fragment.
// There is no split-K: every element of C is summed by one wave in one fixed order, which
// makes a replayed tile bit-identical.
//
// Under this load the device runs against its power limit (the clock settles near 1.85 GHz),
// so bytes moved cost time even when nothing waits for them: the loop issues one LDS read or
// one global load next to each MFMA and nothing else.
//
// Guard: the tile is computed in registers and written once at the end, so a
// work-group may give up at any K step without side effects. The preempt word is
// checked at entry and then every kPollSteps K steps: wave 0 requests it with a vector load
// at the top of the step and looks at it in front of the barrier the loop has anyway, so
// nobody waits for it; a flushed tile leaves its progress byte untagged and is redone by
// the replay. The tile is written out through LDS (64-bit stores of four rows of a column,
// transposing reads back), whole rows of 128 bytes per eight lanes.
// Work-group ids are remapped so that the 32 CUs of one XCD (ids equal modulo 8 land on one
// XCD) work on neighbouring tiles and share A/B panels in that XCD's L2.
#include <type_traits>

#include "hip_hal.h"
#include "xsched/hip/hal.h"

using namespace xsched::preempt;

namespace xsched::hip
{

namespace gemm
{

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4 LdsS16x4;
typedef __attribute__((address_space(3))) void LdsVoid;
typedef __attribute__((address_space(3))) volatile uint32_t LdsVolatileWord;
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kLargeTile = 256;     // edge of the large tile of C (M and N)
constexpr int kSmallTile = 128;     // edge of the small one
constexpr int kStepK = 64;          // K per step
constexpr int kPollSteps = 4;       // K steps between two looks at the preempt word
constexpr int kXcds = 8;
constexpr int kGroupRows = 4;       // tile rows walked together
constexpr int kMaxK = 1 << 22;      // 32-bit byte offsets inside a 256-row panel of A

/// Two floats rounded to nearest-even bf16 (NaNs quieted), `lo` in the low half: the
/// conversion instruction of gfx950 (v_cvt_pk_bf16_f32), which gives bit for bit what the
/// integer formula (u + 0x7FFF + ((u >> 16) & 1)) >> 16, NaN -> (u >> 16) | 0x40 gives (a GPU
/// test compares the two over products that hit ties, overflow, denormals, infinities and
/// NaNs).
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_rne(float lo, float hi)
{
    const bf16x2 pair = __builtin_convertvector(f32x2 { lo, hi }, bf16x2);
    return __builtin_bit_cast(uint32_t, pair);
}

// Work-group id -> tile coordinates. Ids with equal (id % 8) run on one XCD; each
// XCD gets a contiguous run of tiles, ordered in bands of kGroupRows tile rows.
__device__ __forceinline__ void TileOf(uint32_t wg, uint32_t tiles_m, uint32_t tiles_n,
                                       uint32_t &tm, uint32_t &tn)
{
    const uint32_t n_tiles = tiles_m * tiles_n;
    uint32_t t = wg;
    if (n_tiles % kXcds == 0) {
        const uint32_t per_xcd = n_tiles / kXcds;
        t = (wg % kXcds) * per_xcd + wg / kXcds;
    }
    const uint32_t band = kGroupRows * tiles_n;
    const uint32_t band_id = t / band;
    const uint32_t first_row = band_id * kGroupRows;
    const uint32_t rows = min((uint32_t)kGroupRows, tiles_m - first_row);
    const uint32_t in_band = t - band_id * band;
    tm = first_row + in_band % rows;
    tn = in_band / rows;
}

// The compiler keeps the instructions of one group in the order the groups are listed:
// mask 0x008 = MFMA, 0x100 = LDS read.
#define XS_GROUP(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
#define XS_PIN __builtin_amdgcn_sched_barrier(0)
#define XS_WAIT_GLOBAL_LOADS __builtin_amdgcn_s_waitcnt(0x0F70) /* vmcnt(0), nothing else */

// Two LDS buffers and ONE barrier per K step. While the MFMAs of step t read buffer t % 2,
// tile t + 1 is landing in the other buffer (its loads were issued a whole step earlier);
// after the barrier buffer t % 2 is free and the loads of tile t + 2 go out, one next to
// each MFMA of the step's last k slice. The fragments of the next 16-wide k slice are read
// from LDS next to the MFMAs of the current slice, one read per MFMA.
//
// kTile x kTile is the tile of C, kWavesM x kWavesN the wave grid over it; a wave owns
// kBlocksM x kBlocksN blocks of 32x32. Two shapes are built: 256 with 2x4 waves (4x2 blocks
// per wave), and 128 with 2x2 waves (2x2 blocks) for outputs of too few large tiles to fill
// the device. Every element is summed in the same order in both.
//
// (The body is a device function: the host pass cannot parse the buffer-resource builtins
// and would silently drop the launch stub of a kernel that uses them directly.)
template <bool kGuard, int kTile, int kWavesM, int kWavesN>
__device__ __forceinline__
void GemmBf16Body(const uint16_t *__restrict__ A, const uint16_t *__restrict__ B,
                  uint16_t *__restrict__ C, int M, int N, int K, const XGuardArgs &g)
{
    constexpr int kWaves = kWavesM * kWavesN;
    constexpr int kBlocksM = kTile / (32 * kWavesM);
    constexpr int kBlocksN = kTile / (32 * kWavesN);
    constexpr int kMfmas = kBlocksM * kBlocksN;          // per wave and 16-wide k slice
    constexpr int kABytes = kTile * kStepK * 2;          // one A tile in LDS
    constexpr int kBBytes = kStepK * kTile * 2;          // one B tile
    constexpr int kALoads = kABytes / 1024 / kWaves;     // wave-wide 1 KiB loads per wave and tile
    constexpr int kBLoads = kBBytes / 1024 / kWaves;
    constexpr int kLoadsPerMfma = (kALoads + kBLoads) / kMfmas;
    constexpr int kBRowBytes = kTile * 2;                // one k row of the B tile
    constexpr int kBSlotsPerRow = kBRowBytes / 16;
    constexpr int kBRowsPerLoad = 64 / kBSlotsPerRow;
    constexpr uint32_t kBGranuleMask = kBRowBytes / 64 - 1;
    static_assert(kBlocksN == 2, "the block index is XORed into the granule number as one bit");
    static_assert(kMfmas * kLoadsPerMfma == kALoads + kBLoads && kBlocksM + kBlocksN <= kMfmas, "loads and reads pair up with the MFMAs of a slice");
    // One LDS object for everything, the word the waves agree on a poll through included:
    // with a second object the compiler attaches alias scopes to the LDS accesses and then
    // makes every fragment read wait for all global loads that are on their way into LDS.
    __shared__ __attribute__((aligned(1024))) uint8_t lds[2 * (kABytes + kBBytes) + 16];
    uint32_t &guard_word = *(uint32_t *)(lds + 2 * (kABytes + kBBytes));
    uint8_t *const As0 = lds;
    uint8_t *const Bs0 = lds + 2 * kABytes;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave / kWavesN;
    const uint32_t wn = wave % kWavesN;

    uint32_t tm, tn;
    TileOf(blockIdx.x, (uint32_t)M / kTile, (uint32_t)N / kTile, tm, tn);
    const size_t m0 = (size_t)tm * kTile, n0 = (size_t)tn * kTile;

    // ---- global -> LDS: lane l of wave-wide load q fills LDS slot 64 q + l (16 bytes) ----
    // Byte offsets of what each lane fetches, relative to the first element of the tile.
    uint32_t a_off[kALoads], b_off[kBLoads];
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
        const uint32_t q = wave * kALoads + i;
        const uint32_t line = 4 * q + (lane >> 4);
        const uint32_t piece = (lane & 15) ^ (line & 15);   // which piece of the line belongs in this slot
        const uint32_t row = 2 * line + (piece >> 3), kc = piece & 7;
        a_off[i] = (row * (uint32_t)K + kc * 8) * 2;
    }
#pragma unroll
    for (int i = 0; i < kBLoads; ++i) {
        const uint32_t q = wave * kBLoads + i;
        const uint32_t k = kBRowsPerLoad * q + lane / kBSlotsPerRow;
        const uint32_t slot = lane % kBSlotsPerRow;
        const uint32_t granule = (slot >> 2) ^ (((k & 3) | ((k >> 1) & 4)) & kBGranuleMask);
        b_off[i] = (k * (uint32_t)N + granule * 32 + (slot & 3) * 8) * 2;
    }
    const uint16_t *const a_tile = A + m0 * (size_t)K;   // + 64 columns per step
    const uint16_t *const b_tile = B + n0;               // + 64 rows per step

    // Load number idx (A first, then B) of the tile of K step `step` into buffer `buf`.
    auto load_piece = [&](int buf, int step, int idx) {
        if (idx < kALoads) {
            const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void *)(a_tile + (size_t)step * kStepK), 0, 0x7fffffff, 0x00020000);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (LdsVoid *)(As0 + buf * kABytes + (wave * kALoads + idx) * 1024), 16, a_off[idx], 0, 0, 0);
        } else {
            const int i = idx - kALoads;
            const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void *)(b_tile + (size_t)step * kStepK * N), 0, 0x7fffffff, 0x00020000);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (LdsVoid *)(Bs0 + buf * kBBytes + (wave * kBLoads + i) * 1024), 16, b_off[i], 0, 0, 0);
        }
    };
    auto load_tile = [&](int buf, int step) {
#pragma unroll
        for (int idx = 0; idx < kALoads + kBLoads; ++idx) load_piece(buf, step, idx);
    };

    // ---- LDS -> fragments ----
    // A: lane reads row a_row0 + 32 i, pieces 2 ks + (lane >> 5). 32 rows further is 16 lines
    // further: the same swizzle bits, so one base address serves all blocks of the wave.
    const uint32_t a_row0 = 32 * kBlocksM * wm + (lane & 31);
    const uint32_t a_line = a_row0 >> 1;
    const uint32_t a_base = a_line * 256 + (((((lane & 1) << 3) | (lane >> 5)) ^ (a_line & 15)) << 4);
    auto read_a = [&](int buf, int ks, int i) {
        return *(const bf16x8 *)(As0 + buf * kABytes + (a_base ^ (ks << 5)) + i * 4096);
    };
    // B sits in LDS as it sits in memory, [k][n]. The transposing read hands lane l of every 16
    // lanes the element (l & 3) of what lanes 4 * j + (l >> 2), j = 0..3, of the same 16 point
    // at: with lane r pointing at row (r >> 2), columns 4 * (r & 3) .. + 3, lane l receives
    // column l of rows 0..3. Two reads give the eight consecutive k of one fragment. The rows
    // a lane points at all have the same swizzle bits (k & 3 and bit 3 of k are fixed per lane).
    const uint32_t b_row = 8 * (lane >> 5) + ((lane & 15) >> 2);
    const uint32_t b_swz = (((lane & 15) >> 2) | ((lane >> 5) << 2)) & kBGranuleMask;
    const uint32_t b_base = b_row * kBRowBytes + (((kBlocksN * wn) ^ b_swz) << 6) + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
    auto read_b = [&](int buf, int ks, int j) {
        const uint8_t *p = Bs0 + buf * kBBytes + ks * 16 * kBRowBytes + (b_base ^ (j << 6));
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS16x4 *)p);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS16x4 *)(p + 4 * kBRowBytes));
        return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };
    auto read_frags = [&](int buf, int ks, bf16x8 *fa, bf16x8 *fb) {
#pragma unroll
        for (int i = 0; i < kBlocksM; ++i) fa[i] = read_a(buf, ks, i);
#pragma unroll
        for (int j = 0; j < kBlocksN; ++j) fb[j] = read_b(buf, ks, j);
    };

    f32x16 acc[kBlocksM][kBlocksN];
#pragma unroll
    for (int i = 0; i < kBlocksM; ++i)
#pragma unroll
        for (int j = 0; j < kBlocksN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int steps = K / kStepK;
    load_tile(0, 0);

    if (kGuard) {
        XGuardBlock guard(g, blockIdx.x, &guard_word);
        if (!guard.Enter()) {
            XS_WAIT_GLOBAL_LOADS; // nothing may still be on its way into LDS when the group is gone
            return;
        }
    }

    XS_WAIT_GLOBAL_LOADS;
    __syncthreads();
    load_tile(1, steps > 1 ? 1 : 0);

    bf16x8 fa[2][kBlocksM], fb[2][kBlocksN];
    read_frags(0, 0, fa[0], fb[0]);

    // One k slice: the MFMAs on fragment set `set`, the reads of the next slice into the other
    // set, one read after each of the first MFMAs (the small tile has fewer MFMAs than reads:
    // there a B fragment's two reads follow one MFMA).
    auto slice = [&](int set, int next_buf, int next_ks) {
        XS_PIN;
        read_frags(next_buf, next_ks, fa[set ^ 1], fb[set ^ 1]);
#pragma unroll
        for (int i = 0; i < kBlocksM; ++i)
#pragma unroll
            for (int j = 0; j < kBlocksN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][i], fb[set][j], acc[i][j], 0, 0, 0);
        constexpr int kReads = kBlocksM + 2 * kBlocksN;
        if constexpr (kMfmas >= kReads) {
#pragma unroll
            for (int n = 0; n < kReads; ++n) { XS_GROUP(0x008, 1); XS_GROUP(0x100, 1); }
        } else {
#pragma unroll
            for (int n = 0; n < kBlocksM; ++n) { XS_GROUP(0x008, 1); XS_GROUP(0x100, 1); }
#pragma unroll
            for (int n = 0; n < kBlocksN; ++n) { XS_GROUP(0x008, 1); XS_GROUP(0x100, 2); }
        }
        XS_PIN;
    };

    // One K step. The polling form (every kPollSteps-th step of a guarded launch) is a body of
    // its own: its branches split the step into several scheduling regions and put the address
    // arithmetic of the loads behind the barrier, which costs the step about 3 % - paid on one
    // step in kPollSteps instead of on all of them. The last two steps have nothing left to
    // load (`loading` false), the last one nothing to read ahead either (`reading_ahead`
    // false): after its barrier no wave touches the tile buffers any more. False: the
    // work-group has to leave.
    auto step = [&](int t, auto polling, auto loading, auto reading_ahead) -> bool {
        constexpr bool kPoll = decltype(polling)::value;
        constexpr bool kLoad = decltype(loading)::value;
        constexpr bool kReadAhead = decltype(reading_ahead)::value;
        const int cur = t & 1;
        // Wave 0 asks for the preempt word here, with a vector load that is on its way during
        // the whole step, and looks at it just before the barrier: no wave ever waits for the
        // word alone (a scalar load at the barrier made wave 0 wait for the uncached round trip
        // and for all of its LDS reads while the other seven waves stood at the barrier).
        uint32_t polled = 0;
        if (kPoll && wave == 0) polled = xguard_read_flag_begin(xguard_flag_copy(g, blockIdx.x));

        slice(0, cur, 1);
        slice(1, cur, 2);
        slice(0, cur, 3);

        if (kPoll && wave == 0) {
            const bool current = xguard_read_flag_end(polled) == g.epoch;
            if (lane == 0) {
                if (!current) xguard_note_flush(g);
                guard_word = current ? 1u : 0u;
            }
        }
        XS_WAIT_GLOBAL_LOADS; // this wave's part of tile t + 1 has landed
        __syncthreads();      // tile t + 1 is complete, nobody reads buffer cur any more
        if (kPoll) {
            if (*(LdsVolatileWord *)&guard_word == 0) return false; // the whole group leaves together; nothing was written, no load is in flight
        }

        // Last slice of the step: its MFMAs, next to them the first fragments of tile t + 1
        // and the loads of tile t + 2 into the buffer that has just become free.
        XS_PIN;
#pragma unroll
        for (int i = 0; i < kBlocksM; ++i)
#pragma unroll
            for (int j = 0; j < kBlocksN; ++j) {
                const int n = i * kBlocksN + j;
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[1][i], fb[1][j], acc[i][j], 0, 0, 0);
                if (kReadAhead) {
                    if (n < kBlocksM) fa[0][n] = read_a(cur ^ 1, 0, n);
                    else if (n < kBlocksM + kBlocksN) fb[0][n - kBlocksM] = read_b(cur ^ 1, 0, n - kBlocksM);
                }
                if (kLoad) {
#pragma unroll
                    for (int l = 0; l < kLoadsPerMfma; ++l) load_piece(cur, t + 2, n * kLoadsPerMfma + l);
                }
                XS_PIN;
            }
        return true;
    };
    constexpr std::true_type yes {};
    constexpr std::false_type no {};

    const int loading_steps = steps - 2; // steps whose tile t + 2 exists
    if constexpr (!kGuard) {
        for (int t = 0; t < loading_steps; ++t) step(t, no, yes, yes);
    } else {
        for (int t0 = 0; t0 < loading_steps; t0 += kPollSteps) {
            const int last = min(t0 + kPollSteps, loading_steps) - 1;
            for (int t = t0; t < last; ++t) step(t, no, yes, yes);
            if (!step(last, yes, yes, yes)) return;
        }
    }
    if (steps >= 2) step(steps - 2, no, no, yes);
    step(steps - 1, no, no, no);

    // Write-out. A lane holds one column of sixteen rows of each 32x32 block (four runs of four
    // consecutive rows), so storing from the accumulators would mean 2-byte stores to sixteen
    // different rows. Instead every wave turns its strips of 32 rows x 64 columns over in LDS,
    // in an area of its own inside the tile buffers (nobody reads those any more, and nothing
    // is on its way into them): a run of four rows of one column goes in as ONE 64-bit store
    // (the strip is kept column-major, a column padded from 64 to 72 bytes so that the 32
    // columns of a store fall into 32 different 8-byte bank groups), and the transposing read
    // brings it back out row-major: pointed at four rows of columns 8 q + j (lane 4 j + q of
    // every 16), it hands lane l row (l & 3) of columns 8 (l >> 2) + 0..3; a second read four
    // columns further completes 16 bytes per lane, and 8 rows x 128 bytes leave per store.
    constexpr int kStripColumnBytes = 64 + 8;
    constexpr int kStripBytes = 64 * kStripColumnBytes;
    static_assert(2 * kABytes >= kWaves * kStripBytes, "the A buffers hold one strip per wave");
    uint8_t *const strip = As0 + wave * kStripBytes;
    const uint32_t put_at = (lane & 31) * kStripColumnBytes + 4 * (lane >> 5) * 2;
    const uint32_t l16 = lane & 15, patch = lane >> 4;   // a patch: 4 rows x 32 columns per 16 lanes
    const uint32_t get_row = 4 * (patch >> 1), get_col = 32 * (patch & 1);
    const uint32_t get_at = (get_col + 8 * (l16 & 3) + (l16 >> 2)) * kStripColumnBytes + get_row * 2;
#pragma unroll
    for (int i = 0; i < kBlocksM; ++i) {
#pragma unroll
        for (int j = 0; j < kBlocksN; ++j) {
#pragma unroll
            for (int run = 0; run < 4; ++run) {
                const uint32_t lo = f32x2_to_bf16x2_rne(acc[i][j][4 * run], acc[i][j][4 * run + 1]);
                const uint32_t hi = f32x2_to_bf16x2_rne(acc[i][j][4 * run + 2], acc[i][j][4 * run + 3]);
                *(u32x2 *)(strip + 32 * j * kStripColumnBytes + put_at + 8 * run * 2) = u32x2 { lo, hi };
            }
        }
        const size_t row0 = m0 + 32 * kBlocksM * wm + 32 * i;
        const size_t col0 = n0 + 64 * wn + get_col + 8 * (l16 >> 2);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint8_t *p = strip + get_at + 8 * q * 2;
            const s16x4 left = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS16x4 *)p);
            const s16x4 right = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS16x4 *)(p + 4 * kStripColumnBytes));
            const s16x8 row = __builtin_shufflevector(left, right, 0, 1, 2, 3, 4, 5, 6, 7);
            // (non-temporal: C is written once and not read again; left in L2 it pushes out A and B panels
            // that the XCD's other tiles still need: 1 % of the kernel)
            __builtin_nontemporal_store(row, (s16x8 *)(C + (row0 + 8 * q + get_row + (l16 & 3)) * (size_t)N + col0));
        }
    }

    if (kGuard) {
        XGuardBlock guard(g, blockIdx.x, &guard_word);
        guard.Commit();
    }
}

template <bool kGuard, int kTile, int kWavesM, int kWavesN>
__global__ __launch_bounds__(64 * kWavesM * kWavesN)
void GemmBf16Kernel(const uint16_t *__restrict__ A, const uint16_t *__restrict__ B,
                    uint16_t *__restrict__ C, int M, int N, int K, XGuardArgs g)
{
    GemmBf16Body<kGuard, kTile, kWavesM, kWavesN>(A, B, C, M, N, K, g);
}


// Any shape: M, N, K >= 1, any alignment of the three matrices to two bytes. 64 x 64 tiles of
// C, four waves of one 32x32 block each, K in steps of 32 (two slices of 16 through the same
// MFMA as above and in the same order, so an element is summed as the kernels above sum it;
// what lies beyond K is zero). Every load and store is checked against the matrix; a thread's
// eight neighbouring elements come as one 16-byte load where they lie inside the matrix and
// are aligned, one by one otherwise. The loads of the next step are on their way while the
// current one is multiplied. This kernel is the fall-back for the shapes the fast kernels do
// not take, 5-20 times slower than they are. The guard is at entry only: a tile is short.
constexpr int kAnyTile = 64;
constexpr int kAnyK = 32;

template <bool kGuard>
__global__ __launch_bounds__(256)
void GemmBf16AnyShapeKernel(const uint16_t *__restrict__ A, const uint16_t *__restrict__ B,
                            uint16_t *__restrict__ C, int M, int N, int K, uint32_t tiles_n, uint32_t first_wg,
                            XGuardArgs g)
{
    // a row of 32 k values padded to 40: 80-byte rows, every 16-byte fragment aligned
    __shared__ __attribute__((aligned(16))) uint16_t a_rows[kAnyTile][kAnyK + 8];
    __shared__ __attribute__((aligned(16))) uint16_t b_cols[kAnyTile][kAnyK + 8];   // B transposed: [column][k]
    __shared__ uint32_t guard_word;

    XGuardBlock guard(g, first_wg + blockIdx.x, &guard_word);   // its progress bytes follow the fast kernel's
    if (kGuard && !guard.Enter()) return;

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1;
    const size_t m0 = (size_t)(blockIdx.x / tiles_n) * kAnyTile, n0 = (size_t)(blockIdx.x % tiles_n) * kAnyTile;
    const size_t Ms = (size_t)M, Ns = (size_t)N, Ks = (size_t)K;

    // loads of a step: thread t takes A[m0 + t / 4][k0 + 8 (t % 4) + 0..7] and
    // B[k0 + t / 8][n0 + 8 (t % 8) + 0..7]
    const uint32_t a_row = tid >> 2, a_k = (tid & 3) * 8;
    const uint32_t b_k = tid >> 3, b_col = (tid & 7) * 8;
    union Eight { u32x4 v; uint16_t e[8]; };
    auto load_eight = [](const uint16_t *base, size_t first, size_t end, bool row_inside) {
        Eight r;
        r.v = u32x4 { 0, 0, 0, 0 };
        if (!row_inside || first >= end) return r;
        const uint16_t *p = base + first;
        if (first + 8 <= end && (((uintptr_t)p) & 15) == 0) {
            r.v = *(const u32x4 *)p;
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) r.e[i] = first + i < end ? p[i] : (uint16_t)0;
        }
        return r;
    };
    auto load_a = [&](size_t k0) { return load_eight(A + (m0 + a_row) * Ks, k0 + a_k, Ks, m0 + a_row < Ms); };
    auto load_b = [&](size_t k0) { return load_eight(B + (k0 + b_k) * Ns, n0 + b_col, Ns, k0 + b_k < Ks); };

    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;

    Eight a = load_a(0), b = load_b(0);
    for (size_t k0 = 0; k0 < Ks; k0 += kAnyK) {
        __syncthreads();   // the fragments of the previous step have been read
        *(u32x4 *)&a_rows[a_row][a_k] = a.v;
#pragma unroll
        for (int i = 0; i < 8; ++i) b_cols[b_col + i][b_k] = b.e[i];
        __syncthreads();
        if (k0 + kAnyK < Ks) { a = load_a(k0 + kAnyK); b = load_b(k0 + kAnyK); }
        // lane l: A[row l % 32][k 8 (l / 32) + 0..7], B[k 8 (l / 32) + 0..7][column l % 32], per slice of 16
#pragma unroll
        for (int kk = 0; kk < kAnyK; kk += 16) {
            const bf16x8 fa = *(const bf16x8 *)&a_rows[32 * wm + (lane & 31)][kk + 8 * (lane >> 5)];
            const bf16x8 fb = *(const bf16x8 *)&b_cols[32 * wn + (lane & 31)][kk + 8 * (lane >> 5)];
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb, acc, 0, 0, 0);
        }
    }

    // accumulator 4 run + r of lane l: row 8 run + 4 (l / 32) + r, column l % 32 of the block
    const size_t col = n0 + 32 * wn + (lane & 31);
    if (col < Ns) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const size_t row = m0 + 32 * wm + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
            if (row < Ms) C[row * Ns + col] = (uint16_t)f32x2_to_bf16x2_rne(acc[i], 0.0f);
        }
    }
    if (kGuard) guard.Commit();
}

/// Rows [0, rows_fast) of C go to the fast kernel with tiles of fast_tile (rows_fast is then a
/// multiple of it and the shape one the fast kernel takes), rows [rows_fast, M) to the any-shape
/// kernel; either part may be empty. The progress map holds the fast kernel's tiles first.
class HipGemmCommand final : public HipGuardedCommand
{
public:
    HipGemmCommand(const void *A, const void *B, void *C, int M, int N, int K, int rows_fast, int fast_tile, int guard_mode)
        : HipGuardedCommand(FastTiles(rows_fast, N, fast_tile) + AnyTiles(M - rows_fast, N), guard_mode)
        , A_((const uint16_t *)A), B_((const uint16_t *)B), C_((uint16_t *)C), M_(M), N_(N), K_(K)
        , rows_fast_(rows_fast), fast_tile_(fast_tile) {}

    static uint32_t FastTiles(int rows, int N, int tile) { return rows > 0 ? (uint32_t)(rows / tile) * (uint32_t)(N / tile) : 0u; }
    static uint32_t AnyTiles(int rows, int N)
    {
        return rows > 0 ? (uint32_t)((rows + kAnyTile - 1) / kAnyTile) * (uint32_t)((N + kAnyTile - 1) / kAnyTile) : 0u;
    }

protected:
    virtual hipError_t LaunchKernel(hipStream_t stream, bool guarded, const XGuardArgs &g) override
    {
        const uint32_t fast_tiles = FastTiles(rows_fast_, N_, fast_tile_), any_tiles = AnyTiles(M_ - rows_fast_, N_);
        const hipEvent_t stop = TakeStopEvent();   // for the command's last kernel
        if (fast_tiles != 0) {
            const hipEvent_t mine = any_tiles == 0 ? stop : nullptr;
            const dim3 grid(fast_tiles);
            if (fast_tile_ == kLargeTile) {
                const dim3 block(512);
                if (guarded) LaunchWithStop(mine, (GemmBf16Kernel<true, kLargeTile, 2, 4>), grid, block, stream, A_, B_, C_, rows_fast_, N_, K_, g);
                else         LaunchWithStop(mine, (GemmBf16Kernel<false, kLargeTile, 2, 4>), grid, block, stream, A_, B_, C_, rows_fast_, N_, K_, g);
            } else {
                const dim3 block(256);
                if (guarded) LaunchWithStop(mine, (GemmBf16Kernel<true, kSmallTile, 2, 2>), grid, block, stream, A_, B_, C_, rows_fast_, N_, K_, g);
                else         LaunchWithStop(mine, (GemmBf16Kernel<false, kSmallTile, 2, 2>), grid, block, stream, A_, B_, C_, rows_fast_, N_, K_, g);
            }
            const hipError_t err = hipGetLastError();
            if (err != hipSuccess || any_tiles == 0) return err;
        }
        const dim3 grid(any_tiles), block(256);
        const uint32_t tiles_n = (uint32_t)((N_ + kAnyTile - 1) / kAnyTile);
        const uint16_t *a = A_ + (size_t)rows_fast_ * (size_t)K_;
        uint16_t *c = C_ + (size_t)rows_fast_ * (size_t)N_;
        const int rows = M_ - rows_fast_;
        if (guarded) LaunchWithStop(stop, GemmBf16AnyShapeKernel<true>, grid, block, stream, a, B_, c, rows, N_, K_, tiles_n, fast_tiles, g);
        else         LaunchWithStop(stop, GemmBf16AnyShapeKernel<false>, grid, block, stream, a, B_, c, rows, N_, K_, tiles_n, fast_tiles, g);
        return hipGetLastError();
    }

private:
    const uint16_t *A_, *B_;
    uint16_t *C_;
    const int M_, N_, K_;
    const int rows_fast_, fast_tile_;
};

/// The tile edge for an M x N output: large tiles do more arithmetic per byte read from LDS,
/// but each one keeps a single compute unit busy, so an output of few large tiles leaves most
/// of the device idle. Small tiles when the large ones would cover at most half of the compute
/// units, or when M or N is no multiple of the large edge. XSCHED_HIP_GEMM_TILE=128|256
/// overrides the choice where the shape allows.
inline int TileFor(int M, int N);

/// Whether the fast kernels take the shape and the pointers.
inline bool FastKernelsTake(const void *A, const void *B, const void *C, int M, int N, int K)
{
    return M % kSmallTile == 0 && N % kSmallTile == 0 && K % kStepK == 0 && K <= kMaxK && N <= kMaxK &&
           (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15) == 0;
}

inline int TileFor(int M, int N)
{
    const bool large_fits = M % kLargeTile == 0 && N % kLargeTile == 0;
    if (!large_fits) return kSmallTile;
    int64_t forced = 0;
    if (GetEnvInt64("XSCHED_HIP_GEMM_TILE", forced) && (forced == kSmallTile || forced == kLargeTile)) return (int)forced;
    static const int cus = []() {
        int dev = 0, n = 256;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
        return n > 0 ? n : 256;
    }();
    const int64_t large_tiles = (int64_t)(M / kLargeTile) * (N / kLargeTile);
    return large_tiles * 2 <= cus ? kSmallTile : kLargeTile;
}

} // namespace gemm

} // namespace xsched::hip

using namespace xsched::hip;

EXPORT_C_FUNC XResult HipGemmBf16CommandCreate(HwCommandHandle *cmd, const void *A, const void *B,
                                               void *C, int M, int N, int K, int guard)
{
    if (cmd == nullptr || A == nullptr || B == nullptr || C == nullptr || guard < 0 || guard > 3) {
        return kXSchedErrorInvalidValue;
    }
    if (M <= 0 || N <= 0 || K <= 0 || (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 1) != 0) {
        XWARN("HipGemmBf16CommandCreate: M, N and K must be positive and the matrices aligned to their elements (got %d %d %d)", M, N, K);
        return kXSchedErrorInvalidValue;
    }
    // The fast kernels take M and N in multiples of 128, K in multiples of 64 (K and N at most
    // 2^22) and matrices aligned to 16 bytes. Where only M stands in the way, they take the
    // rows up to the last multiple of 128 and the any-shape kernel the rest (the rows of a
    // row-major matrix can be cut anywhere); every other shape goes to the any-shape kernel whole.
    int64_t forced = 0;
    const bool force_any = GetEnvInt64("XSCHED_HIP_GEMM_TILE", forced) && forced == gemm::kAnyTile;
    const int whole_rows = M / gemm::kSmallTile * gemm::kSmallTile;
    int rows_fast = 0;
    if (!force_any && whole_rows > 0 && gemm::FastKernelsTake(A, B, C, whole_rows, N, K)) rows_fast = whole_rows;
    const int fast_tile = rows_fast > 0 ? gemm::TileFor(rows_fast, N) : gemm::kSmallTile;
    // one progress-map byte per tile
    const uint64_t tiles = (uint64_t)gemm::HipGemmCommand::FastTiles(rows_fast, N, fast_tile) +
                           (uint64_t)((M - rows_fast + gemm::kAnyTile - 1) / gemm::kAnyTile) * (uint64_t)((N + gemm::kAnyTile - 1) / gemm::kAnyTile);
    if (tiles > GuardState::kMaxWorkGroups) {
        XWARN("HipGemmBf16CommandCreate: %d x %d needs more than 2^18 tiles", M, N);
        return kXSchedErrorInvalidValue;
    }
    *cmd = HwCommandManager::Add(std::make_shared<gemm::HipGemmCommand>(A, B, C, M, N, K, rows_fast, fast_tile, guard));
    return kXSchedSuccess;
}
