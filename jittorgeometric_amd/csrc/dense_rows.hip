// Dense feature transform of the conv layers on the matrix cores:
//
//     out[V,N] = x1[V,K1] @ W1[K1,N]  (+ x2[V,K2] @ W2[K2,N])  (+ bias[N])
//
// (x @ self.weight in gcn_conv.py:95; out @ weight1 + x @ root_weight + bias in
// sage_conv.py:186-190, which the second operand and the bias row fold into one pass).
// V is 10^5 .. 10^7, K and N are a few hundred at most: the weights fit in LDS and the
// kernel streams the rows of x once.
//
// fp32 in, fp32 accumulate: v_mfma_f32_16x16x4_f32.  A wavefront owns 16 rows of x and 128
// output columns (8 accumulator tiles).  Lane l = 16 * kg + i holds, for row i and every pair
// of steps (q, q + 1), q even, the eight consecutive floats x[i][16 q + 8 kg .. + 7]: two
// 16-byte loads straight from global memory, issued together, so that the four lanes of a
// row ask for a whole 128-byte line at one time.  Register e of step q is the A operand of
// the product over k = 32 (q / 2) + 8 kg + 4 (q % 2) + e.  The B operand of that product for column tile t is
// W[k][column(t, i)] with column(t, i) = 4 i + t (t < 4) or 64 + 4 i + (t - 4): the four
// tiles' values are adjacent in a row of W, so two 16-byte LDS reads fetch the eight B
// operands of a step, and the accumulators of a lane (rows 4 kg + r, its 8 columns) leave as
// two 16-byte stores per row.  The order in which k is walked differs from the natural one;
// a sum's terms are the same.
//
// Work is bound by the fp32 matrix rate (157 TFLOP/s: 209 us for V = 10^6, K = N = 128) and
// by the 1 GB the rows move, about equally; sharing a read of the rows between two products
// does not pay at this arithmetic intensity, which is why the weight gradient keeps its own
// pass.
#include <mutex>

#include "common.h"

namespace jg {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kDenseCols = 128;      // output columns per workgroup (8 tiles of 16)
constexpr int kDenseRows = 16;       // rows per wavefront tile
constexpr int kDenseMaxK = 256;      // K1 + K2

// what a lane loads when its four k lie past K1 + K2: nothing is done to a loaded value before it
// enters the matrix unit, so a wavefront never waits on a load it has just issued
static __device__ __align__(16) float dense_zeros[4];

struct DenseArgs {
    const float *x1, *x2;      // [V,K1], [V,K2] (x2 NULL when K2 == 0)
    const float *w1, *w2;      // [K1,N], [K2,N]
    const float *bias;         // [N] or NULL
    float *out;                // [V,N]
    int V, K1, K2, N;
    int relu;                  // the result is clamped at zero (a layer's activation in the store)
};

// KQ = 16-float steps held in registers (K1 + K2 <= 16 * KQ); WAVES per workgroup
template <int KQ, int WAVES>
__global__ __launch_bounds__(WAVES *kWave) void dense_rows(DenseArgs a)
{
    static_assert(KQ % 2 == 0, "steps are loaded in pairs");
    extern __shared__ float w_lds[];      // [16 * KQ][kDenseCols], zero where k or the column is outside
    const int lane = lane_id();
    const int i = lane & 15, kg = lane >> 4;
    const int col0 = blockIdx.y * kDenseCols;
    const int K = a.K1 + a.K2;

    // ---- weights of this column group into LDS ---------------------------------
    for (int e = threadIdx.x; e < 16 * KQ * (kDenseCols / 4); e += WAVES * kWave) {
        const int k = e / (kDenseCols / 4), c4 = (e % (kDenseCols / 4)) * 4;
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        if (k < K) {
            const float *row = k < a.K1 ? a.w1 + (size_t)k * a.N : a.w2 + (size_t)(k - a.K1) * a.N;
#pragma unroll
            for (int c = 0; c < 4; c++)
                if (col0 + c4 + c < a.N) v[c] = row[col0 + c4 + c];
        }
        *reinterpret_cast<f32x4 *>(w_lds + k * kDenseCols + c4) = v;
    }
    __syncthreads();

    const int tiles = (a.V + kDenseRows - 1) / kDenseRows;
    const int stride = gridDim.x * WAVES;
    int tile = blockIdx.x * WAVES + wave_in_block();

    // this lane's 4 floats of step q of a tile: from x1 while their k lies below K1, then from x2
    auto load_step = [&](int t, int q) -> f32x4 {
        const int row = min(t * kDenseRows + i, a.V - 1);
        const int k = 32 * (q >> 1) + 8 * kg + 4 * (q & 1);
        const float *src = k < a.K1 ? a.x1 + (size_t)row * a.K1 + k : a.x2 + (size_t)row * a.K2 + (k - a.K1);
        return __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(k < K ? src : dense_zeros));
    };
    // the eight B operands of product step (q, e): W[k][4 i .. 4 i + 3] and W[k][64 + 4 i ..], k as above
    const float *w_lane = w_lds + (8 * kg) * kDenseCols + 4 * i;
    auto weights = [&](int step, f32x4 &lo, f32x4 &hi) {
        const int q = step >> 2;
        const float *p = w_lane + (32 * (q >> 1) + 4 * (q & 1) + (step & 3)) * kDenseCols;
        lo = *reinterpret_cast<const f32x4 *>(p);
        hi = *reinterpret_cast<const f32x4 *>(p + 64);
    };

    const int cl = col0 + 4 * i, ch = col0 + 64 + 4 * i;      // this lane's two runs of four columns
    f32x4 bl = {0.f, 0.f, 0.f, 0.f}, bh = {0.f, 0.f, 0.f, 0.f};
    if (a.bias) {
        if (cl < a.N) bl = *reinterpret_cast<const f32x4 *>(a.bias + cl);
        if (ch < a.N) bh = *reinterpret_cast<const f32x4 *>(a.bias + ch);
    }
    f32x4 cur[KQ];
    if (tile < tiles) {
#pragma unroll
        for (int q = 0; q < KQ; q++) cur[q] = load_step(tile, q);
    }
    for (; tile < tiles; tile += stride) {
        const int after = min(tile + stride, tiles - 1);      // past the end: the last tile again, unused
        f32x4 acc[8];
#pragma unroll
        for (int t = 0; t < 8; t++) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        f32x4 lo, hi;
        weights(0, lo, hi);
#pragma unroll
        for (int q = 0; q < KQ; q++) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                // the next step's weights are on their way while this step's products issue
                f32x4 lo_n = lo, hi_n = hi;
                if (4 * q + e + 1 < 4 * KQ) weights(4 * q + e + 1, lo_n, hi_n);
                __builtin_amdgcn_sched_barrier(0);      // the reads leave before the products, not after
                const float av = cur[q][e];
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, lo[t], acc[t], 0, 0, 0);
                    acc[4 + t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, hi[t], acc[4 + t], 0, 0, 0);
                }
                lo = lo_n;
                hi = hi_n;
                __builtin_amdgcn_sched_barrier(0);
            }
            // these registers are free once their products have issued: the next tile's rows
            // start to arrive a whole tile ahead, at no cost in registers
            if (q & 1) {
                cur[q - 1] = load_step(after, q - 1);
                cur[q] = load_step(after, q);
            }
            __builtin_amdgcn_sched_barrier(0);
        }

        // accumulator r of tile t is out[row0 + 4 kg + r][column(t, i)]
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int row = tile * kDenseRows + 4 * kg + r;
            if (row < a.V) {
                float *dst = a.out + (size_t)row * a.N;
                f32x4 lo4 = {acc[0][r] + bl[0], acc[1][r] + bl[1], acc[2][r] + bl[2], acc[3][r] + bl[3]};
                f32x4 hi4 = {acc[4][r] + bh[0], acc[5][r] + bh[1], acc[6][r] + bh[2], acc[7][r] + bh[3]};
                if (a.relu) {
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        lo4[c] = fmaxf(lo4[c], 0.f);
                        hi4[c] = fmaxf(hi4[c], 0.f);
                    }
                }
                if (cl < a.N) __builtin_nontemporal_store(lo4, reinterpret_cast<f32x4 *>(dst + cl));
                if (ch < a.N) __builtin_nontemporal_store(hi4, reinterpret_cast<f32x4 *>(dst + ch));
            }
        }
    }
}

template <int KQ, int WAVES> static void launch_dense(const DenseArgs &a, hipStream_t s)
{
    constexpr size_t lds = (size_t)16 * KQ * kDenseCols * sizeof(float);
    // once per instantiation, whichever thread gets here first (the attribute belongs to the
    // function, not to the call)
    static std::once_flag raised;
    if (lds > 64 * 1024)
        std::call_once(raised, [] {
            (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&dense_rows<KQ, WAVES>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        });
    const int tiles = (a.V + kDenseRows - 1) / kDenseRows;
    const int per_cu = (int)((160 * 1024) / lds) > 0 ? (int)((160 * 1024) / lds) : 1;
    int blocks = 256 * (per_cu > 2 ? 2 : per_cu);
    const int needed = (tiles + WAVES - 1) / WAVES;
    if (blocks > needed) blocks = needed;
    const int groups = (a.N + kDenseCols - 1) / kDenseCols;
    hipLaunchKernelGGL((dense_rows<KQ, WAVES>), dim3((unsigned)blocks, (unsigned)groups), dim3(WAVES * kWave), lds, s, a);
}

}  // namespace jg

using namespace jg;

// 1 when the kernel covers the shape: K1, K2, N multiples of 4, K1 + K2 <= 256
extern "C" __attribute__((visibility("default"))) int32_t jgamd_dense_rows_supported(int32_t K1, int32_t K2, int32_t N)
{
    return K1 > 0 && K2 >= 0 && N > 0 && K1 % 4 == 0 && K2 % 4 == 0 && N % 4 == 0 && K1 + K2 <= kDenseMaxK ? 1 : 0;
}

extern "C" __attribute__((visibility("default"))) int32_t jgamd_dense_rows(const float *x1, const float *w1, int32_t K1,
                                                                           const float *x2, const float *w2, int32_t K2,
                                                                           const float *bias, float *out, int32_t V,
                                                                           int32_t N, int32_t flags, void *stream)
{
    if (V < 0) return fail(JGAMD_ERR_SIZE, "dense_rows: negative V");
    if (flags & ~JGAMD_ROW_RELU) return fail(JGAMD_ERR_SIZE, "dense_rows: unknown flags %d", flags);
    if (!jgamd_dense_rows_supported(K1, K2, N))
        return fail(JGAMD_ERR_UNSUPPORTED, "dense_rows: K1=%d K2=%d N=%d (multiples of 4, K1 + K2 <= %d)", K1, K2, N,
                    kDenseMaxK);
    if (V == 0) return 0;
    if (!x1 || !w1 || !out || (K2 > 0 && (!x2 || !w2))) return fail(JGAMD_ERR_NULL, "dense_rows: NULL array");
    if ((((uintptr_t)x1 | (uintptr_t)x2 | (uintptr_t)out | (uintptr_t)bias) & 15) != 0 ||
        (((uintptr_t)w1 | (uintptr_t)w2) & 3) != 0)
        return fail(JGAMD_ERR_ALIGN, "dense_rows: x / out / bias must be 16-byte aligned");
    const DenseArgs a{x1, K2 > 0 ? x2 : nullptr, w1, K2 > 0 ? w2 : nullptr, bias, out, V, K1, K2 > 0 ? K2 : 0, N,
                      (flags & JGAMD_ROW_RELU) ? 1 : 0};
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int K = a.K1 + a.K2;
    if (K <= 64) launch_dense<4, 8>(a, s);
    else if (K <= 128) launch_dense<8, 8>(a, s);
    else if (K <= 192) launch_dense<12, 8>(a, s);
    else launch_dense<16, 8>(a, s);
    return launch_status("dense_rows");
}
