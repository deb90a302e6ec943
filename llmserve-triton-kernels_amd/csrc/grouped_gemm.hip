// Products with a weight per group:  out[m, g_out + n] = sum_k x[m, g_x + k] * w[g][n][k]
//   groups as column blocks   every row meets every group; group g reads the columns g * x_gs .. + K of x and writes
//                             the columns g * out_gs .. of out (a product per head)
//   groups as row segments    rows seg[g] .. seg[g + 1] belong to group g (rows sorted by expert); a workgroup finds
//                             its group and tile from tile_start[g] = tiles of all groups before g
// Epilogues: plain; "paired" for a weight whose rows alternate between two projections a, b of a gated unit:
// out[m, n / 2] = min(a, limit) * sigmoid(1.702 min(a, limit)) * (clamp(b, -limit, limit) + 1); "gated": the result
// times sigmoid(z[m, g * z_gs + n]) with z in 32-bit.
// This file holds the 32-bit multiply-add kernel (any sizes, float or bfloat16 operands, 32-bit products and sums).
#include "common.h"

#define GG_TM 64
#define GG_TN 64
#define GG_TK 16

#define GG_PLAIN 0
#define GG_PAIRED 1
#define GG_GATED 2

template <typename TIn, typename TOut, int EPI>
__global__ __launch_bounds__(256) void grouped_fma_kernel(
    TOut* __restrict__ out, long out_ld, long out_gs, const TIn* __restrict__ x, long x_ld, long x_gs,
    const TIn* __restrict__ w, int M, int N, int K, int G, const int* __restrict__ seg, const int* __restrict__ tile_start,
    const float* __restrict__ z, long z_ld, long z_gs, float limit) {
    __shared__ float As[GG_TK][GG_TM + 4];
    __shared__ float Ws[GG_TK][GG_TN + 4];
    const int tid = threadIdx.x;
    int g, row0, row_end;
    if (seg) {
        const int t = blockIdx.y;
        if (t >= tile_start[G]) return;
        g = 0;
        while (tile_start[g + 1] <= t) ++g;  // (uniform over the workgroup)
        row0 = seg[g] + (t - tile_start[g]) * GG_TM;
        row_end = seg[g + 1];
    } else {
        g = blockIdx.z;
        row0 = blockIdx.y * GG_TM;
        row_end = M;
    }
    const int n0 = blockIdx.x * GG_TN;
    const TIn* xg = x + (seg ? 0 : (size_t)g * x_gs);
    const TIn* wg = w + (size_t)g * N * K;
    const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
    const int lr = tid / 4, lk = (tid % 4) * 4;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += GG_TK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + lk + i;
            const int am = row0 + lr, wn = n0 + lr;
            As[lk + i][lr] = (am < row_end && k < K) ? to_f32(xg[(size_t)am * x_ld + k]) : 0.f;
            Ws[lk + i][lr] = (wn < N && k < K) ? to_f32(wg[(size_t)wn * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GG_TK; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[k][tm + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Ws[k][tn + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
    TOut* og = out + (seg ? 0 : (size_t)g * out_gs);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = row0 + tm + i;
        if (m >= row_end) continue;
        if (EPI == GG_PAIRED) {
#pragma unroll
            for (int j = 0; j < 4; j += 2) {
                const int n = n0 + tn + j;
                if (n + 1 >= N) continue;
                // (the operands of the second product are rounded as a stored activation would be)
                const float a = fminf(round_to<TOut>(acc[i][j]), limit);
                const float b = fminf(fmaxf(round_to<TOut>(acc[i][j + 1]), -limit), limit);
                og[(size_t)m * out_ld + n / 2] = from_f32<TOut>(a / (1.f + expf(-1.702f * a)) * (b + 1.f));
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = n0 + tn + j;
                if (n >= N) continue;
                float v = acc[i][j];
                if (EPI == GG_GATED) v = v / (1.f + expf(-z[(size_t)m * z_ld + (size_t)g * z_gs + n]));
                og[(size_t)m * out_ld + n] = from_f32<TOut>(v);
            }
        }
    }
}

template <typename TIn, typename TOut>
static int launch_fma(int epilogue, dim3 grid, hipStream_t stream, void* out, long out_ld, long out_gs, const void* x, long x_ld,
                      long x_gs, const void* w, int M, int N, int K, int G, const int* seg, const int* tile_start, const float* z,
                      long z_ld, long z_gs, float limit) {
#define GG_GO(EPI)                                                                                                          \
    grouped_fma_kernel<TIn, TOut, EPI><<<grid, 256, 0, stream>>>((TOut*)out, out_ld, out_gs, (const TIn*)x, x_ld, x_gs,      \
                                                                 (const TIn*)w, M, N, K, G, seg, tile_start, z, z_ld, z_gs, limit)
    if (epilogue == GG_PLAIN) GG_GO(GG_PLAIN);
    else if (epilogue == GG_PAIRED) GG_GO(GG_PAIRED);
    else GG_GO(GG_GATED);
#undef GG_GO
    LLMS_LAUNCH_CHECK();
}

extern "C" {

// in_dtype / out_dtype: 0 = float32, 1 = bfloat16; (0,0), (1,1), (1,0).  `seg` null: groups as column blocks over all
// M rows; else groups as row segments and `max_tiles` workgroups in the grid's second dimension (at least
// tile_start[G], which the host bounds by ceil(M / 64) + G).
int llms_grouped_fma(int in_dtype, int out_dtype, int epilogue, void* out, long out_ld, long out_gs, const void* x, long x_ld,
                     long x_gs, const void* w, int M, int N, int K, int G, const int* seg, const int* tile_start,
                     int max_tiles, const float* z, long z_ld, long z_gs, float limit, hipStream_t stream) {
    LLMS_REQUIRE(M > 0 && N > 0 && K > 0 && G > 0, "grouped_fma: sizes must be positive");
    LLMS_REQUIRE(epilogue >= 0 && epilogue <= 2, "grouped_fma: epilogue 0 (plain), 1 (paired) or 2 (gated)");
    LLMS_REQUIRE(epilogue != GG_PAIRED || N % 2 == 0, "grouped_fma: a paired weight has an even number of rows");
    LLMS_REQUIRE(epilogue != GG_GATED || z, "grouped_fma: the gated epilogue needs its gate products");
    LLMS_REQUIRE((seg == nullptr) == (tile_start == nullptr), "grouped_fma: segments come with their tile starts");
    dim3 grid((N + GG_TN - 1) / GG_TN, seg ? max_tiles : (M + GG_TM - 1) / GG_TM, seg ? 1 : G);
    LLMS_REQUIRE(grid.y > 0 && grid.y <= 65535 && grid.z <= 65535, "grouped_fma: too many rows or groups for one launch");
    if (in_dtype == 0 && out_dtype == 0)
        return launch_fma<float, float>(epilogue, grid, stream, out, out_ld, out_gs, x, x_ld, x_gs, w, M, N, K, G, seg, tile_start,
                                        z, z_ld, z_gs, limit);
    if (in_dtype == 1 && out_dtype == 1)
        return launch_fma<bf16, bf16>(epilogue, grid, stream, out, out_ld, out_gs, x, x_ld, x_gs, w, M, N, K, G, seg, tile_start, z,
                                      z_ld, z_gs, limit);
    if (in_dtype == 1 && out_dtype == 0)
        return launch_fma<bf16, float>(epilogue, grid, stream, out, out_ld, out_gs, x, x_ld, x_gs, w, M, N, K, G, seg, tile_start, z,
                                       z_ld, z_gs, limit);
    LLMS_REQUIRE(false, "grouped_fma: unsupported dtype pair");
}

}  // extern "C"
