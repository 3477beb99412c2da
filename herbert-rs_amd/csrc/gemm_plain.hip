// Plain tiled matrix product in float32 arithmetic for any storage types and any sizes:
//   C[m, n] (+)= sum_k A[m, k] * W[n, k]      (weights are [out, in], k contiguous)
// It is the whole matrix path of the float32 mode and the fallback of the bfloat16
// mode for shapes its MFMA kernels refuse. Each output is summed over k ascending by
// one thread with fused multiply-adds, so its value does not depend on M, on the tile
// it falls in, or on what else is in the batch. (hb_gemm_plain_short_k is the entry for products with a
// short k: it sends up to 32 float32 rows times bfloat16 rows to gemm_few_rows_kernel, whose four partial
// sums a column differ from that order by float32 rounding, and everything else here.)
// In xigh/herbert-rs: crates/backends/backend_bf16/src/kernels.rs:154-164 (float32 sums over k ascending of
// x[m, k] * float(w[n, k]), no bias); crates/backends/backend_vulkan/shaders/bf16_matmul.comp:31-60.
#include "common.h"

HB_MODULE_ERROR_SLOT()

#define TILE_M 64
#define TILE_N 64
#define TILE_K 16

// What a product may do to a sum before it stores it: nothing (rate null), or turn the pre-activation of a
// decay into the decay itself, exp(-exp(rate[n / D]) * softplus(sum + bias[n])) for column n (float32; the
// arithmetic of hb_channel_decay, which does the same to rows that lie in memory). A decay of the other kind
// (rate == bias, the mark of it): sigmoid(sum + bias[n])^root = exp(-root * softplus(-(sum + bias[n]))).
struct DecayEpilogue {
    const float* rate;
    const float* bias;
    int D;
    float root;
};

__device__ __forceinline__ float decay_of(const DecayEpilogue& ep, float sum, int n) {
    const float a = sum + ep.bias[n];
    if (ep.rate == ep.bias) {
        const float softplus = -a > 20.f ? -a : log1pf(expf(-a));
        return expf(-ep.root * softplus);
    }
    const float softplus = a > 20.f ? a : log1pf(expf(a));
    return expf(-expf(ep.rate[n / ep.D]) * softplus);
}

template <class TA, class TW, class TC, bool ACCUM>
__global__ void __launch_bounds__(256)
gemm_plain_kernel(const TA* __restrict__ A, const TW* __restrict__ W, TC* __restrict__ C, int M, int N,
                  int K, int lda, int ldw, int ldc, size_t batch_a, size_t batch_w, size_t batch_c,
                  DecayEpilogue ep) {
    // (blockIdx.z: one of a batch of products whose operands lie batch_* elements apart)
    A += blockIdx.z * batch_a;
    W += blockIdx.z * batch_w;
    C += blockIdx.z * batch_c;
    __shared__ float As[TILE_K][TILE_M + 1];
    __shared__ float Ws[TILE_K][TILE_N + 1];
    const int tid = threadIdx.x;
    const int tx = tid % 16;   // column group
    const int ty = tid / 16;   // row group
    const int m0 = blockIdx.y * TILE_M;
    const int n0 = blockIdx.x * TILE_N;

    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += TILE_K) {
        // 64 x 16 elements of each operand, 4 per thread; k runs fastest in memory.
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid + i * 256;
            const int kk = e % TILE_K;
            const int rr = e / TILE_K;
            const int k = k0 + kk;
            const int m = m0 + rr;
            const int n = n0 + rr;
            As[kk][rr] = (m < M && k < K) ? hb_to_float(A[(size_t)m * lda + k]) : 0.f;
            Ws[kk][rr] = (n < N && k < K) ? hb_to_float(W[(size_t)n * ldw + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < TILE_K; ++kk) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty + 16 * i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx + 16 * j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty + 16 * i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx + 16 * j;
            if (n >= N) continue;
            const size_t idx = (size_t)m * ldc + n;
            if (ACCUM)
                C[idx] = hb_from_float<TC>(hb_to_float(C[idx]) + acc[i][j]);
            else
                C[idx] = hb_from_float<TC>(ep.rate ? decay_of(ep, acc[i][j], n) : acc[i][j]);
        }
    }
}

template <class TA, class TW, class TC>
static void launch(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw, int ldc,
                   int accumulate, hipStream_t stream, int batch = 1, size_t batch_a = 0, size_t batch_w = 0,
                   size_t batch_c = 0, DecayEpilogue ep = DecayEpilogue{nullptr, nullptr, 1, 0.f}) {
    dim3 grid((N + TILE_N - 1) / TILE_N, (M + TILE_M - 1) / TILE_M, batch);
    if (accumulate)
        gemm_plain_kernel<TA, TW, TC, true><<<grid, 256, 0, stream>>>(
            (const TA*)A, (const TW*)W, (TC*)C, M, N, K, lda, ldw, ldc, batch_a, batch_w, batch_c, ep);
    else
        gemm_plain_kernel<TA, TW, TC, false><<<grid, 256, 0, stream>>>(
            (const TA*)A, (const TW*)W, (TC*)C, M, N, K, lda, ldw, ldc, batch_a, batch_w, batch_c, ep);
}


// Few rows times a matrix of bfloat16 rows with a short k (the second product of a pair through a narrow
// middle, one token a sequence): the tiled kernel above would run N / 64 workgroups with a barrier every
// 16 k. Here a wave takes 16 output columns, four lanes a column, each lane a quarter of k in steps of 8
// (one 16-byte load of the weights' row), for up to 8 rows of A at once, which the wave first copies to
// LDS so that no load waits for another; the four partial sums meet by two lane exchanges. Float32
// arithmetic throughout. A's rows and W's rows must be 16-byte aligned, K in steps of 32 up to FEW_ROWS_K.
#define FEW_ROWS_M 8
#define FEW_ROWS_K 1024
__global__ void __launch_bounds__(HB_WAVE)
gemm_few_rows_kernel(const float* __restrict__ A, const bf16* __restrict__ W, float* __restrict__ C, int M, int N,
                     int K, int lda, int ldw, int ldc, DecayEpilogue ep, size_t batch_a = 0, size_t batch_w = 0,
                     size_t batch_c = 0) {
    // (blockIdx.z: one of a batch of products whose operands lie batch_* elements apart)
    A += blockIdx.z * batch_a;
    W += blockIdx.z * batch_w;
    C += blockIdx.z * batch_c;
    __shared__ __attribute__((aligned(16))) float rows_of_a[FEW_ROWS_M * FEW_ROWS_K];
    const int lane = threadIdx.x;
    const int n = blockIdx.x * 16 + lane / 4;
    const int part = lane % 4;
    const int m0 = blockIdx.y * FEW_ROWS_M;
    const int rows = M - m0 < FEW_ROWS_M ? M - m0 : FEW_ROWS_M;
    const int quarter = K / 4;
    for (int idx = lane; idx < FEW_ROWS_M * quarter; idx += HB_WAVE) {
        const int i = idx / quarter, f = idx % quarter;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (i < rows) v = *(const float4*)(A + (size_t)(m0 + i) * lda + 4 * f);
        *(float4*)&rows_of_a[i * K + 4 * f] = v;
    }
    __syncthreads();
    float acc[FEW_ROWS_M];
#pragma unroll
    for (int i = 0; i < FEW_ROWS_M; ++i) acc[i] = 0.f;
    if (n < N) {
        const bf16* w_row = W + (size_t)n * ldw + part * quarter;
        const float* a_row = rows_of_a + part * quarter;
        for (int k = 0; k < quarter; k += 8) {
            const uint4 packed = *(const uint4*)(w_row + k);
            float w[8];
            w[0] = __uint_as_float(packed.x << 16), w[1] = __uint_as_float(packed.x & 0xffff0000u);
            w[2] = __uint_as_float(packed.y << 16), w[3] = __uint_as_float(packed.y & 0xffff0000u);
            w[4] = __uint_as_float(packed.z << 16), w[5] = __uint_as_float(packed.z & 0xffff0000u);
            w[6] = __uint_as_float(packed.w << 16), w[7] = __uint_as_float(packed.w & 0xffff0000u);
#pragma unroll
            for (int i = 0; i < FEW_ROWS_M; ++i) {
                const float4 lo = *(const float4*)(a_row + i * K + k);
                const float4 hi = *(const float4*)(a_row + i * K + k + 4);
                float s = acc[i];
                s = fmaf(lo.x, w[0], s), s = fmaf(lo.y, w[1], s), s = fmaf(lo.z, w[2], s), s = fmaf(lo.w, w[3], s);
                s = fmaf(hi.x, w[4], s), s = fmaf(hi.y, w[5], s), s = fmaf(hi.z, w[6], s), s = fmaf(hi.w, w[7], s);
                acc[i] = s;
            }
        }
    }
#pragma unroll
    for (int i = 0; i < FEW_ROWS_M; ++i) {
        acc[i] += __shfl_xor(acc[i], 1, HB_WAVE);
        acc[i] += __shfl_xor(acc[i], 2, HB_WAVE);
    }
    // (all four lanes of a column hold its sums: each stores, and first turns into a decay, every fourth row)
    static_assert(FEW_ROWS_M % 4 == 0, "the rows are dealt out to a column's four lanes");
#pragma unroll
    for (int j = 0; j < FEW_ROWS_M / 4; ++j) {
        const float s = part == 0 ? acc[4 * j] : part == 1 ? acc[4 * j + 1] : part == 2 ? acc[4 * j + 2] : acc[4 * j + 3];
        const int i = 4 * j + part;
        if (n < N && i < rows) C[(size_t)(m0 + i) * ldc + n] = ep.rate ? decay_of(ep, s, n) : s;
    }
}

static bool few_rows_takes(const void* A, int a_dtype, const void* W, int w_dtype, int c_dtype, int M, int K, int lda,
                           int ldw, int accumulate) {
    return a_dtype == 0 && w_dtype == 1 && c_dtype == 0 && !accumulate && M <= 32 && K % 32 == 0 && K <= FEW_ROWS_K && lda % 4 == 0 &&
           ldw % 8 == 0 && (uintptr_t)A % 16 == 0 && (uintptr_t)W % 16 == 0;
}

// C[M, N] (+)= A[M, K] * W[N, K]^T with row strides lda, ldw, ldc (in elements).
extern "C" int hb_gemm_plain(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype,
                             int M, int N, int K, int lda, int ldw, int ldc, int accumulate,
                             hipStream_t stream) {
    HB_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: empty problem (M=%d, N=%d, K=%d)", M, N, K);
    HB_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm: a row stride is smaller than its row");
    HB_REQUIRE((M + TILE_M - 1) / TILE_M <= 65535, "gemm: M=%d exceeds the grid", M);
    const int key = a_dtype * 4 + w_dtype * 2 + c_dtype;
    switch (key) {
        case 0: launch<float, float, float>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, stream); break;
        case 1: launch<float, float, bf16>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, stream); break;
        case 2: launch<float, bf16, float>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, stream); break;
        case 3: launch<float, bf16, bf16>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, stream); break;
        case 4: launch<bf16, float, float>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, stream); break;
        case 5: launch<bf16, float, bf16>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, stream); break;
        case 6: launch<bf16, bf16, float>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, stream); break;
        case 7: launch<bf16, bf16, bf16>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, stream); break;
        default: HB_REQUIRE(false, "gemm: unknown dtypes (%d, %d, %d)", a_dtype, w_dtype, c_dtype);
    }
    HB_CHECK_LAUNCH("gemm_plain");
    return 0;
}

// The same product for callers whose k is short (a narrow middle): few rows take the kernel made for them.
// A_log [N / D] and dt_bias [N], both or neither: the sums are a decay's pre-activations, and what is stored is
// the decay a column (float32 in and out, no accumulation). A_log == dt_bias: the decay is
// sigmoid(sum + dt_bias[n])^root instead.
extern "C" int hb_gemm_plain_short_k(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype,
                                     int M, int N, int K, int lda, int ldw, int ldc, int accumulate,
                                     const float* A_log, const float* dt_bias, int D, float root,
                                     hipStream_t stream) {
    HB_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: empty problem (M=%d, N=%d, K=%d)", M, N, K);
    HB_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm: a row stride is smaller than its row");
    HB_REQUIRE((A_log == nullptr) == (dt_bias == nullptr), "gemm: a decay needs its rate and its bias");
    HB_REQUIRE(!A_log || (D > 0 && N % D == 0 && c_dtype == 0 && !accumulate),
               "gemm: a decay is float32, stored and not added, %d columns in heads of %d", N, D);
    const DecayEpilogue ep{A_log, dt_bias, A_log ? D : 1, root};
    if (few_rows_takes(A, a_dtype, W, w_dtype, c_dtype, M, K, lda, ldw, accumulate)) {
        gemm_few_rows_kernel<<<dim3((N + 15) / 16, (M + FEW_ROWS_M - 1) / FEW_ROWS_M), HB_WAVE, 0, stream>>>(
            (const float*)A, (const bf16*)W, (float*)C, M, N, K, lda, ldw, ldc, ep);
        HB_CHECK_LAUNCH("gemm_few_rows");
        return 0;
    }
    if (!A_log) return hb_gemm_plain(A, a_dtype, W, w_dtype, C, c_dtype, M, N, K, lda, ldw, ldc, accumulate, stream);
    HB_REQUIRE((M + TILE_M - 1) / TILE_M <= 65535, "gemm: M=%d exceeds the grid", M);
    switch (a_dtype * 2 + w_dtype) {
        case 0: launch<float, float, float>(A, W, C, M, N, K, lda, ldw, ldc, 0, stream, 1, 0, 0, 0, ep); break;
        case 1: launch<float, bf16, float>(A, W, C, M, N, K, lda, ldw, ldc, 0, stream, 1, 0, 0, 0, ep); break;
        case 2: launch<bf16, float, float>(A, W, C, M, N, K, lda, ldw, ldc, 0, stream, 1, 0, 0, 0, ep); break;
        case 3: launch<bf16, bf16, float>(A, W, C, M, N, K, lda, ldw, ldc, 0, stream, 1, 0, 0, 0, ep); break;
        default: HB_REQUIRE(false, "gemm: unknown dtypes (%d, %d)", a_dtype, w_dtype);
    }
    HB_CHECK_LAUNCH("gemm_plain");
    return 0;
}

// A batch of such products in one launch: product b reads A + b * batch_a, W + b * batch_w and writes
// C + b * batch_c (elements). Heads that each have a matrix of their own are such a batch: the row
// strides let every head's columns lie inside rows that all heads share.
extern "C" int hb_gemm_plain_batched(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype,
                                     int M, int N, int K, int lda, int ldw, int ldc, int batch, size_t batch_a,
                                     size_t batch_w, size_t batch_c, hipStream_t stream) {
    HB_REQUIRE(M > 0 && N > 0 && K > 0 && batch > 0, "gemm: empty problem (M=%d, N=%d, K=%d, batch=%d)", M, N, K, batch);
    HB_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm: a row stride is smaller than its row");
    HB_REQUIRE((M + TILE_M - 1) / TILE_M <= 65535 && batch <= 65535, "gemm: M=%d or batch=%d exceeds the grid", M, batch);
    // few rows (one token a sequence) with a short k: the kernel made for them, a product of the batch a grid's layer
    if (few_rows_takes(A, a_dtype, W, w_dtype, c_dtype, M, K, lda, ldw, 0) && batch_a % 4 == 0 && batch_w % 8 == 0) {
        gemm_few_rows_kernel<<<dim3((N + 15) / 16, (M + FEW_ROWS_M - 1) / FEW_ROWS_M, batch), HB_WAVE, 0, stream>>>(
            (const float*)A, (const bf16*)W, (float*)C, M, N, K, lda, ldw, ldc, DecayEpilogue{nullptr, nullptr, 1, 0.f},
            batch_a, batch_w, batch_c);
        HB_CHECK_LAUNCH("gemm_few_rows_batched");
        return 0;
    }
    const int key = a_dtype * 4 + w_dtype * 2 + c_dtype;
#define HB_BATCHED(TA, TW, TC) launch<TA, TW, TC>(A, W, C, M, N, K, lda, ldw, ldc, 0, stream, batch, batch_a, batch_w, batch_c)
    switch (key) {
        case 0: HB_BATCHED(float, float, float); break;
        case 1: HB_BATCHED(float, float, bf16); break;
        case 2: HB_BATCHED(float, bf16, float); break;
        case 3: HB_BATCHED(float, bf16, bf16); break;
        case 4: HB_BATCHED(bf16, float, float); break;
        case 5: HB_BATCHED(bf16, float, bf16); break;
        case 6: HB_BATCHED(bf16, bf16, float); break;
        case 7: HB_BATCHED(bf16, bf16, bf16); break;
        default: HB_REQUIRE(false, "gemm: unknown dtypes (%d, %d, %d)", a_dtype, w_dtype, c_dtype);
    }
#undef HB_BATCHED
    HB_CHECK_LAUNCH("gemm_plain_batched");
    return 0;
}
