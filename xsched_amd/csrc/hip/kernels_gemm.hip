// Guarded bf16 GEMM for gfx950: C[M,N] = A[M,K] * B[K,N], row-major, fp32
// accumulation in ascending k, bf16 (round-to-nearest-even) output.
//
// MFMA-bound: 2*M*N*K flop. One work-group of 512 threads (8 wavefronts) owns one
// 256x256 tile of C and walks K in steps of 64 through two LDS buffers:
//   global -> registers (tile t+2 is requested while tile t is computed), 128-bit loads for
//                       both operands
//   registers -> LDS    A tile as [256 rows][64 k], rows padded to 72 bf16 so that the 128-bit
//                       fragment reads of 32 consecutive rows fall into distinct banks;
//                       B tile as it sits in memory, [64 k][256 cols], rows padded to 272 bf16;
//                       written to the buffer that is not being read, one barrier per step
//   LDS -> MFMA         v_mfma_f32_32x32x16_bf16; wave (wm, wn) of the 2x4 wave grid
//                       accumulates a 128x64 sub-tile = 4x2 blocks of 32x32
// An MFMA operand wants eight consecutive k per lane. A has them contiguous in memory; for B
// (k is the strided dimension) the transposing LDS read of gfx950, ds_read_b64_tr_b16, turns
// four rows of four columns into four k of one column per lane, two of them per fragment.
// There is no split-K: every element of C is summed by one wave in one fixed order, which
// makes a replayed tile bit-identical.
//
// Guard: the tile is computed in registers and written once at the end, so a
// work-group may give up at any K step without side effects. The preempt word is
// checked at entry and then every kPollSteps K steps: wave 0 requests it with a vector load
// at the top of the step and looks at it in front of the barrier the loop has anyway, so
// nobody waits for it; a flushed tile leaves its progress byte untagged and is redone by
// the replay. The tile is written out through LDS, whole rows of 128 bytes per eight lanes. Work-group ids are remapped so that the 32 CUs of one XCD (ids equal
// modulo 8 land on one XCD) work on neighbouring tiles and share A/B panels in that
// XCD's L2.
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

constexpr int kLargeTile = 256;     // edge of the large tile of C (M and N)
constexpr int kSmallTile = 128;     // edge of the small one
constexpr int kStepK = 64;          // K per step
constexpr int kLdsStride = 72;      // bf16 per row of the A tile in LDS (64 + 8 padding)
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4 LdsS16x4;
constexpr int kPollSteps = 8;       // K steps between two looks at the preempt word
constexpr int kXcds = 8;
constexpr int kGroupRows = 4;       // tile rows walked together

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

/// Round-to-nearest-even to bf16, NaNs quieted: the conversion instruction of gfx950
/// (v_cvt_pk_bf16_f32), which gives bit for bit what the integer formula
/// (u + 0x7FFF + ((u >> 16) & 1)) >> 16, NaN -> (u >> 16) | 0x40 gives (a GPU test compares
/// the two over products that hit ties, overflow, denormals, infinities and NaNs).
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f)
{
    const bf16x2 pair = __builtin_convertvector(f32x2 { f, 0.f }, bf16x2);
    return (uint16_t)__builtin_bit_cast(uint32_t, pair);
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

// Two LDS buffers and ONE barrier per K step: while the MFMAs of step t read buffer
// t % 2, the registers holding tile t + 1 are written to the other buffer and the global
// loads of tile t + 2 are issued; the fragments of the next 16-wide k slice are read from
// LDS before the MFMAs of the current slice are issued.
//
// kTile x kTile is the tile of C, kWavesM x kWavesN the wave grid over it; a wave owns
// kBlocksM x kBlocksN blocks of 32x32. Two shapes are built: 256 with 2x4 waves (4x2 blocks
// per wave), and 128 with 2x2 waves (2x2 blocks) for outputs of too few large tiles to fill
// the device. Every element is summed in the same order in both.
template <bool kGuard, int kTile, int kWavesM, int kWavesN>
__global__ __launch_bounds__(64 * kWavesM * kWavesN)
void GemmBf16Kernel(const uint16_t *__restrict__ A, const uint16_t *__restrict__ B,
                             uint16_t *__restrict__ C, int M, int N, int K, XGuardArgs g)
{
    constexpr int kThreads = 64 * kWavesM * kWavesN;
    constexpr int kBlocksM = kTile / (32 * kWavesM);
    constexpr int kBlocksN = kTile / (32 * kWavesN);
    constexpr int kBStride = kTile + 16;               // bf16 per row of the B tile in LDS: four consecutive rows start in four different 32-byte bank groups
    constexpr int kAChunks = kTile * (kStepK / 8) / kThreads; // 16-byte pieces of the A tile per thread
    constexpr int kBChunks = kStepK * (kTile / 8) / kThreads; // and of the B tile
    static_assert(kBlocksN == 2, "the transposing B reads below cover two 32-column blocks per wave");
    __shared__ __attribute__((aligned(16))) uint16_t As[2][kTile * kLdsStride];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[2][kStepK * kBStride];
    __shared__ uint32_t guard_word;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t wm = wave / kWavesN;
    const uint32_t wn = wave % kWavesN;

    uint32_t tm, tn;
    TileOf(blockIdx.x, (uint32_t)M / kTile, (uint32_t)N / kTile, tm, tn);
    const size_t m0 = (size_t)tm * kTile, n0 = (size_t)tn * kTile;

    u32x4 a_reg[kAChunks];
    u32x4 b_vec[kBChunks];

    auto load_global = [&](int k0) {
#pragma unroll
        for (int i = 0; i < kAChunks; ++i) {
            const uint32_t c = tid + kThreads * i;
            const uint32_t row = c >> 3, kc = c & 7;
            a_reg[i] = *(const u32x4 *)(A + (m0 + row) * (size_t)K + k0 + kc * 8);
        }
#pragma unroll
        for (int i = 0; i < kBChunks; ++i) {
            const uint32_t c = tid + kThreads * i;
            const uint32_t krow = c / (kTile / 8), chunk = c % (kTile / 8);
            b_vec[i] = *(const u32x4 *)(B + (size_t)(k0 + krow) * N + n0 + chunk * 8);
        }
    };

    auto store_lds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < kAChunks; ++i) {
            const uint32_t c = tid + kThreads * i;
            const uint32_t row = c >> 3, kc = c & 7;
            *(u32x4 *)(As[buf] + row * kLdsStride + kc * 8) = a_reg[i];
        }
#pragma unroll
        for (int i = 0; i < kBChunks; ++i) {
            const uint32_t c = tid + kThreads * i;
            const uint32_t krow = c / (kTile / 8), chunk = c % (kTile / 8);
            *(u32x4 *)(Bs[buf] + krow * kBStride + chunk * 8) = b_vec[i];
        }
    };

    const uint32_t a_row0 = 32 * kBlocksM * wm + (lane & 31);
    const uint32_t khalf = 8 * (lane >> 5);
    auto load_a_frags = [&](int buf, int ks, bf16x8 *fa) {
        const uint32_t koff = ks * 16 + khalf;
#pragma unroll
        for (int i = 0; i < kBlocksM; ++i) fa[i] = *(const bf16x8 *)(As[buf] + (a_row0 + 32 * i) * kLdsStride + koff);
    };
    // B sits in LDS as it sits in memory, [k][n]. The transposing read hands lane l of every 16
    // lanes the element (l & 3) of what lanes 4 * j + (l >> 2), j = 0..3, of the same 16 point
    // at: with lane r pointing at row (r >> 2), columns 4 * (r & 3) .. + 3, lane l receives
    // column l of rows 0..3. Two reads give the eight consecutive k of one fragment.
    const uint32_t b_tr_row = 8 * (lane >> 5) + ((lane & 15) >> 2);
    const uint32_t b_tr_col = 64 * wn + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    auto load_b_frags = [&](int buf, int ks, bf16x8 *fb) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint16_t *p = Bs[buf] + (ks * 16 + b_tr_row) * kBStride + b_tr_col + 32 * j;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS16x4 *)p);
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsS16x4 *)(p + 4 * kBStride));
            const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            fb[j] = __builtin_bit_cast(bf16x8, both);
        }
    };
    auto load_frags = [&](int buf, int ks, bf16x8 *fa, bf16x8 *fb) {
        load_a_frags(buf, ks, fa);
        load_b_frags(buf, ks, fb);
    };

    f32x16 acc[kBlocksM][kBlocksN];
#pragma unroll
    for (int i = 0; i < kBlocksM; ++i)
#pragma unroll
        for (int j = 0; j < kBlocksN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    load_global(0);

    if (kGuard) {
        XGuardBlock guard(g, blockIdx.x, &guard_word);
        if (!guard.Enter()) return;
    }

    const int steps = K / kStepK;
    store_lds(0);
    load_global(steps > 1 ? kStepK : 0);
    __syncthreads();

    // The loop body is branch-free (loads and LDS stores past the last tile are clamped or
    // harmless repeats), so that it is one scheduling region. Per step and wave: 32 MFMAs in four k slices of 8; next to them
    //   slice 0: fragment reads of slice 1
    //   slice 1: fragment reads of slice 2, registers of tile t+1 -> the other LDS buffer
    //   slice 2: fragment reads of slice 3, global loads of tile t+2
    //   barrier  (the other buffer is complete, this one is no longer read)
    //   slice 3: fragment reads of slice 0 of the NEXT tile from the other buffer
    // Both fragment sets are double-buffered in registers (40 of them): the reads of slice
    // s + 1 are issued before the MFMAs of slice s.
    bf16x8 fa[2][kBlocksM], fb[2][kBlocksN];
    load_frags(0, 0, fa[0], fb[0]);

    auto mfma_slice = [&](int set) {
#pragma unroll
        for (int i = 0; i < kBlocksM; ++i)
#pragma unroll
            for (int j = 0; j < kBlocksN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][i], fb[set][j], acc[i][j], 0, 0, 0);
    };

    for (int t = 0; t < steps; ++t) {
        const int cur = t & 1;
        const int k_next = (t + 2 < steps ? t + 2 : steps - 1) * kStepK;
        // Every kPollSteps steps wave 0 asks for the preempt word here, with a vector load that
        // is on its way during the whole step, and looks at it just before the barrier: no
        // wave ever waits for the word alone (a scalar load at the barrier made wave 0 wait
        // for the uncached round trip and for all of its LDS reads while the other seven
        // waves stood at the barrier).
        const bool poll_step = kGuard && (t % kPollSteps) == kPollSteps - 1;
        uint32_t polled = 0;
        if (poll_step && wave == 0) polled = xguard_read_flag_begin(xguard_flag_copy(g, blockIdx.x));

        load_frags(cur, 1, fa[1], fb[1]);
        mfma_slice(0);

        load_frags(cur, 2, fa[0], fb[0]);
        store_lds(cur ^ 1);
        mfma_slice(1);

        load_frags(cur, 3, fa[1], fb[1]);
        load_global(k_next);
        mfma_slice(0);

        if (poll_step && wave == 0) {
            const bool current = xguard_read_flag_end(polled) == g.epoch;
            if (lane == 0) {
                if (!current) xguard_note_flush(g);
                guard_word = current ? 1u : 0u;
            }
        }
        __syncthreads(); // buffer cur^1 is complete, buffer cur is free to be overwritten
        if (poll_step) {
            if (guard_word == 0) return; // whole group leaves together; nothing was written
        }

        load_frags(cur ^ 1, 0, fa[0], fb[0]);
        mfma_slice(1);
    }

    // Write-out. A lane holds one column of sixteen rows of each 32x32 block, so storing from
    // the accumulators means 2-byte stores to sixteen different rows. Instead every wave turns
    // its strips of 32 rows x 64 columns over in LDS (an area of its own in the A buffers,
    // rows padded by 8 bf16), and stores them as whole rows: 16 bytes per lane, eight lanes to
    // a row of 128 bytes.
    constexpr int kStripStride = 64 + 8;
    static_assert(sizeof(As) >= (size_t)kWavesM * kWavesN * 32 * kStripStride * 2, "the A buffers hold one strip per wave");
    __syncthreads(); // every wave has read its last fragments
    uint16_t *strip = &As[0][0] + wave * (32 * kStripStride);
#pragma unroll
    for (int i = 0; i < kBlocksM; ++i) {
#pragma unroll
        for (int j = 0; j < kBlocksN; ++j) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                strip[row * kStripStride + 32 * j + (lane & 31)] = f32_to_bf16_rne(acc[i][j][r]);
            }
        }
        const size_t row0 = m0 + 32 * kBlocksM * wm + 32 * i;
        const size_t col0 = n0 + 64 * wn + 8 * (lane & 7);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t row = 8 * q + (lane >> 3);
            const u32x4 v = *(const u32x4 *)(strip + row * kStripStride + 8 * (lane & 7));
            *(u32x4 *)(C + (row0 + row) * (size_t)N + col0) = v;
        }
    }

    if (kGuard) {
        XGuardBlock guard(g, blockIdx.x, &guard_word);
        guard.Commit();
    }
}


class HipGemmCommand final : public HipGuardedCommand
{
public:
    HipGemmCommand(const void *A, const void *B, void *C, int M, int N, int K, int tile, int guard_mode)
        : HipGuardedCommand((uint32_t)(M / tile) * (uint32_t)(N / tile), guard_mode)
        , A_((const uint16_t *)A), B_((const uint16_t *)B), C_((uint16_t *)C), M_(M), N_(N), K_(K), tile_(tile) {}

protected:
    virtual hipError_t LaunchKernel(hipStream_t stream, bool guarded, const XGuardArgs &g) override
    {
        const dim3 grid(n_wg_);
        if (tile_ == kLargeTile) {
            const dim3 block(512);
            if (guarded) hipLaunchKernelGGL((GemmBf16Kernel<true, kLargeTile, 2, 4>), grid, block, 0, stream, A_, B_, C_, M_, N_, K_, g);
            else         hipLaunchKernelGGL((GemmBf16Kernel<false, kLargeTile, 2, 4>), grid, block, 0, stream, A_, B_, C_, M_, N_, K_, g);
        } else {
            const dim3 block(256);
            if (guarded) hipLaunchKernelGGL((GemmBf16Kernel<true, kSmallTile, 2, 2>), grid, block, 0, stream, A_, B_, C_, M_, N_, K_, g);
            else         hipLaunchKernelGGL((GemmBf16Kernel<false, kSmallTile, 2, 2>), grid, block, 0, stream, A_, B_, C_, M_, N_, K_, g);
        }
        return hipGetLastError();
    }

private:
    const uint16_t *A_, *B_;
    uint16_t *C_;
    const int M_, N_, K_;
    const int tile_;
};

/// The tile edge for an M x N output: large tiles do more arithmetic per byte read from LDS,
/// but each one keeps a single compute unit busy, so an output of few large tiles leaves most
/// of the device idle. Small tiles when the large ones would cover at most half of the compute
/// units, or when M or N is no multiple of the large edge. XSCHED_HIP_GEMM_TILE=128|256
/// overrides the choice where the shape allows.
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
    if (M <= 0 || N <= 0 || K <= 0 || M % gemm::kSmallTile || N % gemm::kSmallTile || K % gemm::kStepK) {
        XWARN("HipGemmBf16CommandCreate: M and N must be multiples of 128 and K of 64 (got %d %d %d)", M, N, K);
        return kXSchedErrorInvalidValue;
    }
    const int tile = gemm::TileFor(M, N);
    if ((((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15) != 0) return kXSchedErrorInvalidValue;
    // one progress-map byte per tile
    if ((uint64_t)(M / tile) * (uint64_t)(N / tile) > GuardState::kMaxWorkGroups) {
        return kXSchedErrorInvalidValue;
    }
    *cmd = HwCommandManager::Add(std::make_shared<gemm::HipGemmCommand>(A, B, C, M, N, K, tile, guard));
    return kXSchedSuccess;
}
