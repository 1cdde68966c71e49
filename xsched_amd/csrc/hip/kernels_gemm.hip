// Guarded bf16 GEMM for gfx950: C[M,N] = A[M,K] * B[K,N], row-major, fp32
// accumulation in ascending k, bf16 (round-to-nearest-even) output.
//
// MFMA-bound: 2*M*N*K flop. One work-group of 512 threads (8 wavefronts) owns one
// 256x256 tile of C and walks K in steps of 64:
//   global -> registers (prefetch of step t+1 while step t is computed)
//   registers -> LDS    A tile as [256 rows][64 k], B tile transposed to [256 cols][64 k],
//                       both with rows padded to 72 bf16 so that the 128-bit fragment
//                       reads of 32 consecutive rows fall into distinct banks
//   LDS -> MFMA         v_mfma_f32_32x32x16_bf16; wave (wm, wn) of the 2x4 wave grid
//                       accumulates a 128x64 sub-tile = 4x2 blocks of 32x32
// B is read from global memory as 32-bit words (two columns) over eight k rows and
// transposed in registers with byte permutes, so that LDS holds k-contiguous
// fragments for both operands. There is no split-K: every element of C is summed by
// one wave in one fixed order, which makes a replayed tile bit-identical.
//
// Guard: the tile is computed in registers and written once at the end, so a
// work-group may give up at any K step without side effects. The preempt word is
// checked at entry and then every kPollSteps K steps (piggy-backed on a barrier the
// loop has anyway); a flushed tile leaves its progress bit clear and is redone by
// the replay. Work-group ids are remapped so that the 32 CUs of one XCD (ids equal
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

constexpr int kTile = 256;          // tile edge (M and N)
constexpr int kStepK = 64;          // K per step
constexpr int kLdsStride = 72;      // bf16 per LDS row (64 + 8 padding)
constexpr int kThreads = 512;
constexpr int kPollSteps = 8;       // K steps between two looks at the preempt word
constexpr int kXcds = 8;
constexpr int kGroupRows = 4;       // tile rows walked together

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f)
{
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u); // quiet NaN
    const uint32_t lsb = (u >> 16) & 1u;
    return (uint16_t)((u + 0x7FFFu + lsb) >> 16);
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

template <bool kGuard>
__global__ __launch_bounds__(kThreads)
void GemmBf16Kernel(const uint16_t *__restrict__ A, const uint16_t *__restrict__ B,
                    uint16_t *__restrict__ C, int M, int N, int K, XGuardArgs g)
{
    __shared__ __attribute__((aligned(16))) uint16_t As[kTile * kLdsStride];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[kTile * kLdsStride];
    __shared__ uint32_t guard_word;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t wm = wave >> 2;   // 0..1 : rows 128*wm
    const uint32_t wn = wave & 3;    // 0..3 : cols 64*wn

    uint32_t tm, tn;
    TileOf(blockIdx.x, (uint32_t)M / kTile, (uint32_t)N / kTile, tm, tn);
    const size_t m0 = (size_t)tm * kTile, n0 = (size_t)tn * kTile;

    // ---- global -> register staging -------------------------------------------------
    // A: 256 rows x 8 chunks of 8 bf16 = 2048 chunks, 4 per thread.
    // B: 8 k-groups (of 8 rows) x 128 column pairs = 1024 items, 2 per thread.
    u32x4 a_reg[4];
    uint32_t b_reg[2][8];

    auto load_global = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t c = tid + kThreads * i;
            const uint32_t row = c >> 3, kc = c & 7;
            a_reg[i] = *(const u32x4 *)(A + (m0 + row) * (size_t)K + k0 + kc * 8);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint32_t c = tid + kThreads * i;
            const uint32_t npair = c & 127, kg = c >> 7;
            const uint16_t *src = B + (size_t)(k0 + kg * 8) * N + n0 + npair * 2;
#pragma unroll
            for (int r = 0; r < 8; ++r) b_reg[i][r] = *(const uint32_t *)(src + (size_t)r * N);
        }
    };

    auto store_lds = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t c = tid + kThreads * i;
            const uint32_t row = c >> 3, kc = c & 7;
            *(u32x4 *)(As + row * kLdsStride + kc * 8) = a_reg[i];
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint32_t c = tid + kThreads * i;
            const uint32_t npair = c & 127, kg = c >> 7;
            // b_reg[i][r] = { B[k+r][n] (low half), B[k+r][n+1] (high half) }.
            // Column n gets the low halves of rows r, r+1 packed; column n+1 the high halves.
            u32x4 col0, col1;
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const uint32_t lo = b_reg[i][2 * p], hi = b_reg[i][2 * p + 1];
                col0[p] = __builtin_amdgcn_perm(hi, lo, 0x05040100u); // lo.l | hi.l << 16
                col1[p] = __builtin_amdgcn_perm(hi, lo, 0x07060302u); // lo.h | hi.h << 16
            }
            *(u32x4 *)(Bs + (npair * 2 + 0) * kLdsStride + kg * 8) = col0;
            *(u32x4 *)(Bs + (npair * 2 + 1) * kLdsStride + kg * 8) = col1;
        }
    };

    f32x16 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    load_global(0);

    if (kGuard) {
        XGuardBlock guard(g, blockIdx.x, &guard_word);
        if (!guard.Enter()) return;
    }

    const int steps = K / kStepK;
    for (int t = 0; t < steps; ++t) {
        store_lds();
        if (kGuard && t != 0 && (t % kPollSteps) == 0 && tid == 0) {
            guard_word = xguard_read_flag(xguard_flag_copy(g, blockIdx.x)) == g.epoch ? 1u : 0u;
        }
        __syncthreads();
        if (kGuard && t != 0 && (t % kPollSteps) == 0) {
            if (guard_word == 0) return; // whole group leaves together; nothing was written
        }
        if (t + 1 < steps) load_global((t + 1) * kStepK);

#pragma unroll
        for (int ks = 0; ks < kStepK / 16; ++ks) {
            const uint32_t koff = ks * 16 + 8 * (lane >> 5);
            bf16x8 a_frag[4], b_frag[2];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t row = 128 * wm + 32 * i + (lane & 31);
                a_frag[i] = *(const bf16x8 *)(As + row * kLdsStride + koff);
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const uint32_t col = 64 * wn + 32 * j + (lane & 31);
                b_frag[j] = *(const bf16x8 *)(Bs + col * kLdsStride + koff);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_frag[i], b_frag[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads(); // everyone is done reading before the next store_lds()
    }

    // ---- epilogue: fp32 -> bf16, one store per accumulator register ------------------
    // Accumulator register r of a 32x32 block holds row 8*(r/4) + 4*(lane/32) + r%4,
    // column lane%32.
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const size_t col = n0 + 64 * wn + 32 * j + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const size_t row = m0 + 128 * wm + 32 * i + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                C[row * (size_t)N + col] = f32_to_bf16_rne(acc[i][j][r]);
            }
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
    HipGemmCommand(const void *A, const void *B, void *C, int M, int N, int K, int guard_mode)
        : HipGuardedCommand((uint32_t)(M / kTile) * (uint32_t)(N / kTile), guard_mode)
        , A_((const uint16_t *)A), B_((const uint16_t *)B), C_((uint16_t *)C), M_(M), N_(N), K_(K) {}

protected:
    virtual hipError_t LaunchKernel(hipStream_t stream, bool guarded, const XGuardArgs &g) override
    {
        const dim3 grid(n_wg_), block(kThreads);
        if (guarded) hipLaunchKernelGGL(GemmBf16Kernel<true>, grid, block, 0, stream, A_, B_, C_, M_, N_, K_, g);
        else         hipLaunchKernelGGL(GemmBf16Kernel<false>, grid, block, 0, stream, A_, B_, C_, M_, N_, K_, g);
        return hipGetLastError();
    }

private:
    const uint16_t *A_, *B_;
    uint16_t *C_;
    const int M_, N_, K_;
};

} // namespace gemm

} // namespace xsched::hip

using namespace xsched::hip;

EXPORT_C_FUNC XResult HipGemmBf16CommandCreate(HwCommandHandle *cmd, const void *A, const void *B,
                                               void *C, int M, int N, int K, int guard)
{
    if (cmd == nullptr || A == nullptr || B == nullptr || C == nullptr || guard < 0 || guard > 3) {
        return kXSchedErrorInvalidValue;
    }
    if (M <= 0 || N <= 0 || K <= 0 || M % gemm::kTile || N % gemm::kTile || K % gemm::kStepK) {
        XWARN("HipGemmBf16CommandCreate: M and N must be multiples of 256 and K of 64 (got %d %d %d)", M, N, K);
        return kXSchedErrorInvalidValue;
    }
    if ((((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15) != 0) return kXSchedErrorInvalidValue;
    // one progress-map byte per tile
    if ((uint64_t)(M / gemm::kTile) * (uint64_t)(N / gemm::kTile) > GuardState::kMaxWorkGroups) {
        return kXSchedErrorInvalidValue;
    }
    *cmd = HwCommandManager::Add(std::make_shared<gemm::HipGemmCommand>(A, B, C, M, N, K, guard));
    return kXSchedSuccess;
}
