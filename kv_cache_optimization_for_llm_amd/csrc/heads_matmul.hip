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
                    const T *__restrict__ w, int M, int N, int K, const T *__restrict__ gate, int g_row) {
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
        // (optional) the head's gate: the row's outputs of head h times sigmoid(gate[m, h])
        const float gmul = gate ? 1.0f / (1.0f + expf(-to_float(gate[(size_t)m * g_row + h]))) : 1.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) out[(size_t)m * o_row + (size_t)h * o_head + n] = from_float<T>(acc[i][j] * gmul);
        }
    }
}

extern "C" int kva_heads_matmul(void *out, int o_row, int o_head, const void *x, int x_row, int x_head,
                                const void *w, int rows, int heads, int N, int K, const void *gate, int g_row,
                                int dtype, hipStream_t stream) {
    KVA_REQUIRE(rows >= 0 && heads > 0 && heads <= 65535 && N > 0 && K > 0, "heads_matmul: bad sizes");
    KVA_REQUIRE(x_head >= K && o_head >= N && x_row >= (heads - 1) * x_head + K && o_row >= (heads - 1) * o_head + N,
                "heads_matmul: strides do not fit %d heads of %d -> %d", heads, K, N);
    if (rows == 0) return KVA_OK;
    dim3 grid((N + HM_BN - 1) / HM_BN, (rows + HM_BM - 1) / HM_BM, heads), block(256);
    KVA_REQUIRE(grid.y <= 65535, "heads_matmul: %d rows are too many for one launch", rows);
    if (dtype == KVA_F32)
        hipLaunchKernelGGL(heads_matmul_kernel<float>, grid, block, 0, stream, (float *)out, o_row, o_head,
                           (const float *)x, x_row, x_head, (const float *)w, rows, N, K, (const float *)gate, g_row);
    else if (dtype == KVA_BF16)
        hipLaunchKernelGGL(heads_matmul_kernel<bf16_t>, grid, block, 0, stream, (bf16_t *)out, o_row, o_head,
                           (const bf16_t *)x, x_row, x_head, (const bf16_t *)w, rows, N, K, (const bf16_t *)gate, g_row);
    else KVA_REQUIRE(false, "heads_matmul: unsupported dtype %d", dtype);
    KVA_CHECK_LAUNCH("heads_matmul");
    return KVA_OK;
}

// ---- the same product on the matrix cores (bf16) ------------------------------------------------
//
// A wavefront takes 16 outputs n of one head and walks over tiles of 16 rows t:
// out^T[n, t] = W[h][n, :] . x[t, h, :].  A = 16 rows of W[h] (16 bytes a lane, row-major), kept
// in registers for all the row tiles the wavefront visits; B = x^T: lane (row t, group g) loads 16
// bytes of its row.  K = 32 NKS.  blockIdx: (n tile, head, group of row tiles).
#include "attention_frag.h"

template <int NKS, int NT>
__global__ void __launch_bounds__(KVA_WAVE)
heads_matmul_mfma_kernel(bf16_t *__restrict__ out, int o_row, int o_head, const bf16_t *__restrict__ x, int x_row,
                         int x_head, const bf16_t *__restrict__ w, int M, int N, int tiles_per_wave,
                         const bf16_t *__restrict__ gate, int g_row) {
    // NT neighbouring tiles of 16 outputs a wavefront: every fragment of x it loads serves NT products
    // (many rows: what a wavefront takes in per product is what bounds it); NT = 1 for few rows,
    // where more wavefronts matter more
    constexpr int K = NKS * 32;
    const int lane = threadIdx.x, r = lane & 15, g = lane >> 4;
    const int n_first = blockIdx.x * 16 * NT, h = blockIdx.y;
    Frag8 wf[NT][NKS];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int n = min(n_first + 16 * nt + r, N - 1);
        const bf16_t *wrow = w + ((size_t)h * N + n) * K + 8 * g;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) wf[nt][ks].u4 = *reinterpret_cast<const uint4 *>(wrow + 32 * ks);
    }
    const int first = blockIdx.z * tiles_per_wave;
    for (int tile = first; tile < first + tiles_per_wave && tile * 16 < M; ++tile) {
        const int t = min(tile * 16 + r, M - 1);
        const bf16_t *xrow = x + (size_t)t * x_row + (size_t)h * x_head + 8 * g;
        Frag8 xf[NKS];
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) xf[ks].u4 = *reinterpret_cast<const uint4 *>(xrow + 32 * ks);
        float gmul = 1.f;
        if (gate) gmul = 1.0f / (1.0f + expf(-to_float(gate[(size_t)t * g_row + h])));
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int n0 = n_first + 16 * nt;
            if (n0 >= N) break;
            f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[nt][ks].v, xf[ks].v, acc, 0, 0, 0);
            // lane (row t = r, group g) holds outputs n0 + 4 g .. + 3 of its row
            if (tile * 16 + r < M) {
                bf16_t *o = out + (size_t)t * o_row + (size_t)h * o_head + n0 + 4 * g;
                if (n0 + 4 * g + 3 < N && ((o_row | o_head) % 4 == 0)) {
                    Frag4 v;
#pragma unroll
                    for (int i = 0; i < 4; ++i) v.h[i] = float_to_bf16_bits(acc[i] * gmul);
                    *reinterpret_cast<uint2 *>(o) = v.u2;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (n0 + 4 * g + i < N) o[i].bits = float_to_bf16_bits(acc[i] * gmul);
                }
            }
        }
    }
}

#define HM_INSTANCES(X) X(1) X(2) X(3) X(4) X(6) X(8) X(12) X(16)

extern "C" int kva_heads_matmul_mfma_supported(int K, int x_row, int x_head) {
    if (K % 32 || x_row % 8 || x_head % 8) return 0;
#define CHECK_ONE(NKS) if (K == NKS * 32) return 1;
    HM_INSTANCES(CHECK_ONE)
#undef CHECK_ONE
    return 0;
}

extern "C" int kva_heads_matmul_mfma(void *out, int o_row, int o_head, const void *x, int x_row, int x_head,
                                     const void *w, int rows, int heads, int N, int K, const void *gate, int g_row,
                                     hipStream_t stream) {
    KVA_REQUIRE(rows >= 0 && heads > 0 && heads <= 65535 && N > 0, "heads_matmul_mfma: bad sizes");
    KVA_REQUIRE(kva_heads_matmul_mfma_supported(K, x_row, x_head),
                "heads_matmul_mfma: no instance for K = %d with strides %d / %d", K, x_row, x_head);
    KVA_REQUIRE(x_head >= K && o_head >= N && x_row >= (heads - 1) * x_head + K && o_row >= (heads - 1) * o_head + N,
                "heads_matmul_mfma: strides do not fit %d heads of %d -> %d", heads, K, N);
    if (rows == 0) return KVA_OK;
    const int row_tiles = (rows + 15) / 16;
    const int n_tiles = (N + 15) / 16;
    // many rows: several output tiles a wavefront (at most 32 fragments of W in its registers)
    const bool wide = rows > 64;
    bool done = false;
#define LAUNCH_ONE(NKS)                                                                                          \
    if (!done && K == NKS * 32) {                                                                                \
        constexpr int NTW = NKS <= 8 ? 4 : (NKS <= 16 ? 2 : 1);                                                  \
        const int nt = wide ? NTW : 1;                                                                           \
        const int groups = (n_tiles + nt - 1) / nt;                                                              \
        /* enough wavefronts to fill the chip before a wavefront takes more than one row tile */                 \
        int per_wave = 1;                                                                                        \
        while (per_wave < 8 && (long long)groups * heads * ((row_tiles + per_wave - 1) / per_wave) > 4096) per_wave *= 2; \
        dim3 grid(groups, heads, (row_tiles + per_wave - 1) / per_wave), block(KVA_WAVE);                        \
        KVA_REQUIRE(grid.z <= 65535, "heads_matmul_mfma: %d rows are too many for one launch", rows);            \
        auto kernel = wide ? heads_matmul_mfma_kernel<NKS, NTW> : heads_matmul_mfma_kernel<NKS, 1>;              \
        hipLaunchKernelGGL(kernel, grid, block, 0, stream, (bf16_t *)out, o_row, o_head,                         \
                           (const bf16_t *)x, x_row, x_head, (const bf16_t *)w, rows, N, per_wave,               \
                           (const bf16_t *)gate, g_row);                                                         \
        done = true;                                                                                             \
    }
    HM_INSTANCES(LAUNCH_ONE)
#undef LAUNCH_ONE
    KVA_CHECK_LAUNCH("heads_matmul_mfma");
    return KVA_OK;
}
