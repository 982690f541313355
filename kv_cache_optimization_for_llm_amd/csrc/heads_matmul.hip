// One small matrix product per head: out[t, h, :] = W[h] x[t, h, :] for W [heads, N, K].
//
// It serves projections that differ from head to head (a low-rank key/value entry expanded per
// head, or the same expansion moved to the query side).  x and out are addressed with a row
// stride and a head stride each, so both may be column ranges of wider buffers.  Operands are
// fp32 or bf16; sums are fp32 with k ascending into one accumulator per output, so a row's result
// does not depend on the other rows of the launch.
#include "common.h"

#define HM_BM 64
#define HM_BN 64
#define HM_BK 16

template <typename T>
__global__ void __launch_bounds__(256)
heads_matmul_kernel(T *__restrict__ out, int o_row, int o_head, const T *__restrict__ x, int x_row, int x_head,
                    const T *__restrict__ w, int M, int N, int K) {
    __shared__ float Xs[HM_BK][HM_BM + 4];
    __shared__ float Ws[HM_BK][HM_BN + 4];
    const int h = blockIdx.z;
    const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
    const int m0 = blockIdx.y * HM_BM, n0 = blockIdx.x * HM_BN;
    const int lrow = tid / 4, lk = (tid % 4) * 4;
    const T *xh = x + (size_t)h * x_head, *wh = w + (size_t)h * N * K;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    for (int k0 = 0; k0 < K; k0 += HM_BK) {
        float a[4] = {0.f, 0.f, 0.f, 0.f}, b[4] = {0.f, 0.f, 0.f, 0.f};
        const int am = m0 + lrow, wn = n0 + lrow, kk = k0 + lk;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (am < M && kk + e < K) a[e] = to_float(xh[(size_t)am * x_row + kk + e]);
            if (wn < N && kk + e < K) b[e] = to_float(wh[(size_t)wn * K + kk + e]);
        }
        __syncthreads();
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            Xs[lk + e][lrow] = a[e];
            Ws[lk + e][lrow] = b[e];
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < HM_BK; ++k) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = Xs[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[j] = Ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) out[(size_t)m * o_row + (size_t)h * o_head + n] = from_float<T>(acc[i][j]);
        }
    }
}

extern "C" int kva_heads_matmul(void *out, int o_row, int o_head, const void *x, int x_row, int x_head,
                                const void *w, int rows, int heads, int N, int K, int dtype, hipStream_t stream) {
    KVA_REQUIRE(rows >= 0 && heads > 0 && heads <= 65535 && N > 0 && K > 0, "heads_matmul: bad sizes");
    KVA_REQUIRE(x_head >= K && o_head >= N && x_row >= (heads - 1) * x_head + K && o_row >= (heads - 1) * o_head + N,
                "heads_matmul: strides do not fit %d heads of %d -> %d", heads, K, N);
    if (rows == 0) return KVA_OK;
    dim3 grid((N + HM_BN - 1) / HM_BN, (rows + HM_BM - 1) / HM_BM, heads), block(256);
    KVA_REQUIRE(grid.y <= 65535, "heads_matmul: %d rows are too many for one launch", rows);
    if (dtype == KVA_F32)
        hipLaunchKernelGGL(heads_matmul_kernel<float>, grid, block, 0, stream, (float *)out, o_row, o_head,
                           (const float *)x, x_row, x_head, (const float *)w, rows, N, K);
    else if (dtype == KVA_BF16)
        hipLaunchKernelGGL(heads_matmul_kernel<bf16_t>, grid, block, 0, stream, (bf16_t *)out, o_row, o_head,
                           (const bf16_t *)x, x_row, x_head, (const bf16_t *)w, rows, N, K);
    else KVA_REQUIRE(false, "heads_matmul: unsupported dtype %d", dtype);
    KVA_CHECK_LAUNCH("heads_matmul");
    return KVA_OK;
}
