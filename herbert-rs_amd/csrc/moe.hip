// A feed-forward of many small experts of which each token uses a few.
//   route     the router's logits (+ bias) of a token -> its `top` experts (largest logits, the
//             lower index of equals), weighed by exp(logit) normalised over those experts alone
//   group     the (token, choice) pairs in the order of their experts, so that an expert's rows
//             are consecutive, and a list of row tiles (expert, first row, rows) of fixed length
//   products  a tile's rows times its expert's matrix, float32 sums over k ascending by one
//             thread each (plain), whatever else is in the batch
//   activate  g = min(gate, limit), u = clamp(up, -limit, limit): y = g sigmoid(alpha g) (u + shift)
//             (limit infinite, alpha 1, shift 0: silu(gate) up)
//   combine   a token's rows weighted and summed in the order of its choices, added to the output
// Nothing here asks the host: the grids depend on the step's size only, so a step can be recorded
// and replayed.
#include "common.h"
#include <math.h>

HB_MODULE_ERROR_SLOT()

#define MOE_TILE_M 64
#define MOE_TILE_N 64
#define MOE_TILE_K 16
#define MOE_MAX_E_PER_LANE 16

// ------------------------------------------------------------------------ route
// One wave a token; lane l holds the logits of experts l, l + 64, ...
__global__ void __launch_bounds__(HB_WAVE)
moe_route_kernel(const float* __restrict__ logits, int ld, const float* __restrict__ bias, int* __restrict__ chosen,
                 float* __restrict__ weight, int E, int top) {
    const int t = blockIdx.x, lane = threadIdx.x;
    float z[MOE_MAX_E_PER_LANE];
#pragma unroll
    for (int i = 0; i < MOE_MAX_E_PER_LANE; ++i) {
        const int e = lane + HB_WAVE * i;
        z[i] = e < E ? logits[(size_t)t * ld + e] + (bias ? bias[e] : 0.f) : -INFINITY;
    }
    float first = 0.f, sum = 0.f;
    for (int j = 0; j < top; ++j) {
        float best = -INFINITY;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < MOE_MAX_E_PER_LANE; ++i) {
            const int e = lane + HB_WAVE * i;
            if (e < E && (z[i] > best || (z[i] == best && e < at))) {
                best = z[i];
                at = e;
            }
        }
#pragma unroll
        for (int off = HB_WAVE / 2; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, HB_WAVE);
            const int oa = __shfl_xor(at, off, HB_WAVE);
            if (ob > best || (ob == best && oa < at)) {
                best = ob;
                at = oa;
            }
        }
        if (j == 0) first = best;                    // the first choice is the largest
        const float p = expf(best - first);
        sum += p;
        if (lane == j % HB_WAVE) {                   // (the lane that divides it below)
            chosen[(size_t)t * top + j] = at;
            weight[(size_t)t * top + j] = p;
        }
#pragma unroll
        for (int i = 0; i < MOE_MAX_E_PER_LANE; ++i)
            if (lane + HB_WAVE * i == at) z[i] = -INFINITY;
    }
    for (int j = lane; j < top; j += HB_WAVE) weight[(size_t)t * top + j] /= sum;
}

// Routing by scores s = sigmoid(logit). The choice runs on s + correction, the weights on s itself:
// the experts form n_groups equal runs of adjacent experts, a group is worth the two highest of its
// selection values, added; only the experts of the `keep` best groups can be chosen (the lower index of equals,
// for groups as for experts), and the chosen experts' scores are divided by their sum + 1e-20.
// Three parameters change the form: softmax_scores (s is the softmax of the logits over all E experts instead of
// their sigmoids), worth_top (how many of a group's highest selection values make its worth: 2, or 1), renorm
// (0: the weights are the chosen experts' scores as they are).
// One wave a token; the scores lie in LDS.
__global__ void __launch_bounds__(HB_WAVE)
moe_route_scores_kernel(const float* __restrict__ logits, int ld, const float* __restrict__ correction,
                        int* __restrict__ chosen, float* __restrict__ weight, int E, int top, int n_groups,
                        int keep, int softmax_scores, int worth_top, int renorm) {
    __shared__ float score[HB_WAVE * MOE_MAX_E_PER_LANE];
    __shared__ float choice[HB_WAVE * MOE_MAX_E_PER_LANE];
    __shared__ float worth[HB_WAVE * MOE_MAX_E_PER_LANE];
    __shared__ int kept[HB_WAVE * MOE_MAX_E_PER_LANE];
    const int t = blockIdx.x, lane = threadIdx.x;
    const int size = E / n_groups;
    float top_logit = -INFINITY, denom = 1.0f;
    if (softmax_scores) {
        for (int e = lane; e < E; e += HB_WAVE) top_logit = fmaxf(top_logit, logits[(size_t)t * ld + e]);
        top_logit = hb_wave_max(top_logit);
        float part = 0.f;
        for (int e = lane; e < E; e += HB_WAVE) part += expf(logits[(size_t)t * ld + e] - top_logit);
        denom = hb_wave_sum(part);
    }
    for (int e = lane; e < E; e += HB_WAVE) {
        const float z = logits[(size_t)t * ld + e];
        const float s = softmax_scores ? expf(z - top_logit) / denom : 1.0f / (1.0f + expf(-z));
        score[e] = s;
        choice[e] = s + (correction ? correction[e] : 0.f);
    }
    __syncthreads();
    for (int g = lane; g < n_groups; g += HB_WAVE) {
        float a = -INFINITY, b = -INFINITY;          // the largest and the second
        for (int i = 0; i < size; ++i) {
            const float c = choice[g * size + i];
            if (c > a) {
                b = a;
                a = c;
            } else if (c > b) {
                b = c;
            }
        }
        worth[g] = (size > 1 && worth_top > 1) ? a + b : a;
    }
    __syncthreads();
    for (int g = lane; g < n_groups; g += HB_WAVE) {
        int ahead = 0;
        for (int o = 0; o < n_groups; ++o) ahead += (worth[o] > worth[g] || (worth[o] == worth[g] && o < g)) ? 1 : 0;
        kept[g] = ahead < keep;
    }
    __syncthreads();
    float z[MOE_MAX_E_PER_LANE];
#pragma unroll
    for (int i = 0; i < MOE_MAX_E_PER_LANE; ++i) {
        const int e = lane + HB_WAVE * i;
        z[i] = (e < E && kept[e / size]) ? choice[e] : -INFINITY;
    }
    float sum = 0.f;
    for (int j = 0; j < top; ++j) {
        float best = -INFINITY;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < MOE_MAX_E_PER_LANE; ++i) {
            const int e = lane + HB_WAVE * i;
            // (experts outside the kept groups and those already taken are never met: they are marked below)
            if (e < E && z[i] != -INFINITY && (z[i] > best || at == 0x7fffffff || (z[i] == best && e < at))) {
                best = z[i];
                at = e;
            }
        }
#pragma unroll
        for (int off = HB_WAVE / 2; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, HB_WAVE);
            const int oa = __shfl_xor(at, off, HB_WAVE);
            if (oa != 0x7fffffff && (at == 0x7fffffff || ob > best || (ob == best && oa < at))) {
                best = ob;
                at = oa;
            }
        }
        if (at == 0x7fffffff) at = 0;                // (fewer experts in the kept groups than `top`: the host refuses that)
        const float s = score[at];
        sum += s;
        if (lane == j % HB_WAVE) {
            chosen[(size_t)t * top + j] = at;
            weight[(size_t)t * top + j] = s;
        }
#pragma unroll
        for (int i = 0; i < MOE_MAX_E_PER_LANE; ++i)
            if (lane + HB_WAVE * i == at) z[i] = -INFINITY;
    }
    if (!renorm) return;
    const float total = sum + 1e-20f;
    for (int j = lane; j < top; j += HB_WAVE) weight[(size_t)t * top + j] /= total;
}

// ------------------------------------------------------------------------ group
// Block e < E: the pairs of expert e, in the order of the pairs, to rows [first, first + count) and
// the expert's tiles into the list; block E: the list's unused end. order[row] = pair,
// row_of[pair] = row. Every block counts all experts' pairs for itself (a histogram in LDS), so that
// no kernel has to run before it. Experts from `real` on have no matrices (their output is their input): their
// pairs get rows like any others, but their tiles are marked as holding nothing, so no product runs on them.
__global__ void __launch_bounds__(256)
moe_place_kernel(const int* __restrict__ chosen, int* __restrict__ counts, int* __restrict__ order,
                 int* __restrict__ row_of, int* __restrict__ tile_expert, int* __restrict__ tile_row0,
                 int* __restrict__ tile_rows, int A, int E, int max_tiles, int real) {
    __shared__ int hist[HB_WAVE * MOE_MAX_E_PER_LANE];
    __shared__ int wave_n[4];
    __shared__ int base;
    const int e = blockIdx.x;
    for (int i = threadIdx.x; i < E; i += blockDim.x) hist[i] = 0;
    __syncthreads();
    for (int a = threadIdx.x; a < A; a += blockDim.x) atomicAdd(&hist[chosen[a]], 1);
    __syncthreads();
    int first = 0, tile0 = 0;
    for (int i = 0; i < (e < E ? e : E); ++i) {
        first += hist[i];
        tile0 += (hist[i] + MOE_TILE_M - 1) / MOE_TILE_M;
    }
    if (e == E) {
        for (int i = tile0 + threadIdx.x; i < max_tiles; i += blockDim.x) tile_expert[i] = -1;
        return;
    }
    const int count = hist[e];
    if (threadIdx.x == 0) counts[e] = count;
    for (int i = threadIdx.x; i * MOE_TILE_M < count; i += blockDim.x) {
        tile_expert[tile0 + i] = e < real ? e : -1;
        tile_row0[tile0 + i] = first + i * MOE_TILE_M;
        tile_rows[tile0 + i] = count - i * MOE_TILE_M < MOE_TILE_M ? count - i * MOE_TILE_M : MOE_TILE_M;
    }
    if (count == 0) return;
    if (threadIdx.x == 0) base = first;
    __syncthreads();
    const int lane = threadIdx.x & (HB_WAVE - 1), wave = threadIdx.x / HB_WAVE;
    for (int a0 = 0; a0 < A; a0 += 256) {
        const int a = a0 + threadIdx.x;
        const bool hit = a < A && chosen[a] == e;
        const unsigned long long mask = __ballot(hit);
        if (lane == 0) wave_n[wave] = __popcll(mask);
        __syncthreads();
        int before = 0;
        for (int w = 0; w < wave; ++w) before += wave_n[w];
        if (hit) {
            const int row = base + before + __popcll(mask & ((1ull << lane) - 1ull));
            order[row] = a;
            row_of[a] = row;
        }
        __syncthreads();
        if (threadIdx.x == 0) base += wave_n[0] + wave_n[1] + wave_n[2] + wave_n[3];
        __syncthreads();
    }
}

// logits' rows are ld floats apart (their first E count).
// by_scores 0: the largest logits (+ bias), weights a softmax over the chosen.
// by_scores 1: sigmoid scores, `bias` is the correction of the choice, n_groups groups of which `keep` count.
extern "C" int hb_moe_route(const float* logits, const float* bias, int* chosen, float* weight, int* counts,
                            int* order, int* row_of, int* tile_expert, int* tile_row0, int* tile_rows, int T, int E,
                            int top, int max_tiles, int ld, int by_scores, int n_groups, int keep, int real,
                            int softmax_scores, int worth_top, int renorm, hipStream_t stream) {
    HB_REQUIRE(ld >= E, "moe: logits rows %d apart for %d experts", ld, E);
    HB_REQUIRE(!by_scores || (n_groups > 0 && E % n_groups == 0 && keep > 0 && keep <= n_groups &&
                              top <= keep * (E / n_groups)),
               "moe: %d of %d groups of %d experts cannot give %d experts", keep, n_groups, E, top);
    HB_REQUIRE(T > 0 && E > 0 && top > 0 && top <= E, "moe: %d of %d experts for %d tokens", top, E, T);
    HB_REQUIRE(real > 0 && real <= E, "moe: %d of %d experts have matrices", real, E);
    HB_REQUIRE(E <= HB_WAVE * MOE_MAX_E_PER_LANE, "moe: %d experts, the router takes up to %d", E, HB_WAVE * MOE_MAX_E_PER_LANE);
    const long long A = (long long)T * top;
    HB_REQUIRE(A < (1ll << 30), "moe: too many (token, expert) pairs");
    HB_REQUIRE(max_tiles >= (A + MOE_TILE_M - 1) / MOE_TILE_M + E, "moe: the tile list is too short");
    if (by_scores)
        moe_route_scores_kernel<<<T, HB_WAVE, 0, stream>>>(logits, ld, bias, chosen, weight, E, top, n_groups, keep,
                                                           softmax_scores, worth_top, renorm);
    else
        moe_route_kernel<<<T, HB_WAVE, 0, stream>>>(logits, ld, bias, chosen, weight, E, top);
    HB_CHECK_LAUNCH("moe_route");
    moe_place_kernel<<<E + 1, 256, 0, stream>>>(chosen, counts, order, row_of, tile_expert, tile_row0, tile_rows, (int)A, E, max_tiles, real);
    HB_CHECK_LAUNCH("moe_place");
    return 0;
}

// ------------------------------------------------------------------------ products, plain
// C[row, n] = sum_k A[src(row), k] * W[e][n, k] for the rows of every tile; src(row) = order[row] / top
// (the token's row of the activations) if `top` > 0, else the row itself.
template <class TA, class TW, class TC>
__global__ void __launch_bounds__(256)
moe_gemm_plain_kernel(const TA* __restrict__ A, const TW* __restrict__ W, TC* __restrict__ C,
                      const int* __restrict__ order, const int* __restrict__ tile_expert,
                      const int* __restrict__ tile_row0, const int* __restrict__ tile_rows, int top, int N, int K) {
    __shared__ float As[MOE_TILE_K][MOE_TILE_M + 1];
    __shared__ float Ws[MOE_TILE_K][MOE_TILE_N + 1];
    __shared__ int src[MOE_TILE_M];
    const int e = tile_expert[blockIdx.y];
    if (e < 0) return;
    const int row0 = tile_row0[blockIdx.y], rows = tile_rows[blockIdx.y];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    const int n0 = blockIdx.x * MOE_TILE_N;
    const TW* We = W + (size_t)e * N * K;
    if (tid < MOE_TILE_M) src[tid] = tid < rows ? (top > 0 ? order[row0 + tid] / top : row0 + tid) : -1;
    __syncthreads();

    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += MOE_TILE_K) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int el = tid + i * 256;
            const int kk = el % MOE_TILE_K, rr = el / MOE_TILE_K;
            const int k = k0 + kk, n = n0 + rr;
            As[kk][rr] = (src[rr] >= 0 && k < K) ? hb_to_float(A[(size_t)src[rr] * K + k]) : 0.f;
            Ws[kk][rr] = (n < N && k < K) ? hb_to_float(We[(size_t)n * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < MOE_TILE_K; ++kk) {
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
        const int r = ty + 16 * i;
        if (r >= rows) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx + 16 * j;
            if (n < N) C[(size_t)(row0 + r) * N + n] = hb_from_float<TC>(acc[i][j]);
        }
    }
}

// A [rows, K] (the tokens' rows if top > 0, else one row a pair), W [E, N, K], C [pairs, N].
extern "C" int hb_moe_gemm_plain(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype,
                                 const int* order, const int* tile_expert, const int* tile_row0,
                                 const int* tile_rows, int max_tiles, int top, int N, int K, hipStream_t stream) {
    HB_REQUIRE(N > 0 && K > 0 && max_tiles > 0 && max_tiles <= 65535 * 16, "moe product: empty or too large");
    HB_REQUIRE(max_tiles <= 65535, "moe product: %d row tiles exceed the grid", max_tiles);
    const dim3 grid((N + MOE_TILE_N - 1) / MOE_TILE_N, max_tiles);
    const int key = a_dtype * 4 + w_dtype * 2 + c_dtype;
#define HB_MOE(TA, TW, TC)                                                                                        \
    moe_gemm_plain_kernel<TA, TW, TC><<<grid, 256, 0, stream>>>((const TA*)A, (const TW*)W, (TC*)C, order,        \
                                                                tile_expert, tile_row0, tile_rows, top, N, K)
    switch (key) {
        case 0: HB_MOE(float, float, float); break;
        case 2: HB_MOE(float, bf16, float); break;
        case 4: HB_MOE(bf16, float, float); break;
        case 6: HB_MOE(bf16, bf16, float); break;
        default: HB_REQUIRE(false, "moe product: dtypes (%d, %d, %d) are not built (the sums are float32)", a_dtype, w_dtype, c_dtype);
    }
#undef HB_MOE
    HB_CHECK_LAUNCH("moe_gemm_plain");
    return 0;
}

// ------------------------------------------------------------------------ activate
// gu [pairs, 2 F] float32 (gate columns, then up columns) -> act [pairs, F]
template <class TOut>
__global__ void moe_activate_kernel(const float* __restrict__ gu, TOut* __restrict__ act, int F, size_t total,
                                    float limit, float alpha, float shift) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / F;
        const int n = (int)(i % F);
        const float g = fminf(gu[r * 2 * F + n], limit);
        const float u = fminf(fmaxf(gu[r * 2 * F + F + n], -limit), limit);
        act[i] = hb_from_float<TOut>(g / (1.0f + expf(-alpha * g)) * (u + shift));
    }
}

extern "C" int hb_moe_activate(const float* gu, void* act, int act_dtype, int rows, int F, float limit, float alpha,
                               float shift, hipStream_t stream) {
    HB_REQUIRE(rows > 0 && F > 0, "moe activation: empty input");
    const size_t total = (size_t)rows * F;
    const size_t blocks = (total + 255) / 256;
    const unsigned grid = (unsigned)(blocks > 8192 ? 8192 : blocks);
    if (act_dtype == HB_F32)
        moe_activate_kernel<float><<<grid, 256, 0, stream>>>(gu, (float*)act, F, total, limit, alpha, shift);
    else if (act_dtype == HB_BF16)
        moe_activate_kernel<bf16><<<grid, 256, 0, stream>>>(gu, (bf16*)act, F, total, limit, alpha, shift);
    else
        HB_REQUIRE(false, "moe activation: unknown output dtype %d", act_dtype);
    HB_CHECK_LAUNCH("moe_activate");
    return 0;
}

// ------------------------------------------------------------------------ combine
// x[t, :] += sum_j weight[t, j] * y[row_of[t * top + j], :]    (float32, j ascending)
// shared [T, H] (or null): a part that every token takes, added times sigmoid(gate[t * gate_ld]).
// input [T, H] (or null) with chosen [T, top] and real: a pair whose expert is `real` or beyond has no row in y;
// its output is the token's own input row.
template <class TIn>
__global__ void moe_combine_kernel(const float* __restrict__ y, const float* __restrict__ weight,
                                   const int* __restrict__ row_of, float* __restrict__ x, int top, int H,
                                   const float* __restrict__ shared, const float* __restrict__ gate, int gate_ld,
                                   const TIn* __restrict__ input, const int* __restrict__ chosen, int real) {
    const int t = blockIdx.x;
    const float open = shared ? 1.0f / (1.0f + expf(-gate[(size_t)t * gate_ld])) : 0.f;
    // (a token's rows and weights once, eight at a time, then whole rows)
    for (int j0 = 0; j0 < top; j0 += 8) {
        const float* rows[8];
        float w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const bool in = j0 + j < top;
            rows[j] = y + (size_t)row_of[(size_t)t * top + (in ? j0 + j : 0)] * H;
            w[j] = in ? weight[(size_t)t * top + j0 + j] : 0.f;
            if (input != nullptr && in && chosen[(size_t)t * top + j0 + j] >= real) rows[j] = nullptr;
        }
        for (int i = threadIdx.x; i < H; i += blockDim.x) {
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (j0 + j < top)
                    s = fmaf(w[j], rows[j] != nullptr ? rows[j][i] : hb_to_float(input[(size_t)t * H + i]), s);
            if (shared && j0 == 0) s = fmaf(open, shared[(size_t)t * H + i], s);
            x[(size_t)t * H + i] += s;
        }
    }
}

extern "C" int hb_moe_combine(const float* y, const float* weight, const int* row_of, float* x, int T, int top, int H,
                              const float* shared, const float* gate, int gate_ld, const void* input,
                              int input_dtype, const int* chosen, int real, hipStream_t stream) {
    HB_REQUIRE(shared == nullptr || (gate != nullptr && gate_ld > 0), "moe combine: a shared part needs its gate");
    HB_REQUIRE(T > 0 && top > 0 && H > 0, "moe combine: empty input");
    HB_REQUIRE(input == nullptr || chosen != nullptr, "moe combine: experts without matrices need the choices");
    const int threads = H >= 1024 ? 256 : 64;
    if (input != nullptr && input_dtype == HB_BF16)
        moe_combine_kernel<bf16><<<T, threads, 0, stream>>>(y, weight, row_of, x, top, H, shared, gate, gate_ld,
                                                            (const bf16*)input, chosen, real);
    else
        moe_combine_kernel<float><<<T, threads, 0, stream>>>(y, weight, row_of, x, top, H, shared, gate, gate_ld,
                                                             (const float*)input, chosen, real);
    HB_CHECK_LAUNCH("moe_combine");
    return 0;
}

// ------------------------------------------------------------------------ products on the matrix cores
// The same products for bfloat16 operands with float32 sums (v_mfma_f32_16x16x32_bf16), and more
// generally a group of products that share a shape: group g multiplies rows of A (from column
// g * a_group_off on) with its own matrix W[g] [N, K] into columns of C from g * c_group_off on.
// W[g] is stored in the order of the operands, [K / 32][N / 16][64 lanes][8] (the 1 KB of 16 rows and 32 k
// in a row, lane = 16 (k / 8 % 4) + n % 16): a wave's load is one contiguous KB, where rows K apart
// would each give 64 bytes from addresses a power of two apart.
// The rows of a group come as a list of tiles (group, first row, rows <= 64) or, without a list, as
// every group's ceil(M / 64) tiles of the same M rows (heads that each have a matrix of their own).
// A workgroup is four waves on one tile of 64 rows; a wave holds four blocks of 16 weight rows
// against up to four blocks of 16 activation rows (the blocks beyond the tile's rows are skipped, so
// a tile of a few rows costs little more than streaming its weights). The weights go from memory
// straight into the lanes (lane l of an operand holds 8 consecutive k of row l % 16 from k0 + 8 (l / 16)),
// a stage ahead of their products; the tile's activations, which the four waves share, through two
// stages in LDS.
// An output is summed over k in the same order whatever else the tile holds.
// EPI 0: float32 C. EPI 1: bfloat16 C. EPI 2: W[g] is [2 F, K], gate rows then up rows; a wave's two
// blocks are 16 gate rows and the 16 up rows that go with them, and C [*, F] bfloat16 receives
// min(gate, limit) sigmoid(alpha min(gate, limit)) (clamp(up, -limit, limit) + shift).
typedef __bf16 hb_bf16x8 __attribute__((ext_vector_type(8)));
typedef float hb_f32x4 __attribute__((ext_vector_type(4)));

#define GM_KSTEP 64           // k a stage of the activations' ring in LDS

template <int EPI>
__global__ void __launch_bounds__(256)
grouped_mfma_kernel(const bf16* __restrict__ A, int lda, size_t a_group_off, const bf16* __restrict__ W, int N,
                    int K, void* __restrict__ Cv, int ldc, size_t c_group_off, const int* __restrict__ order,
                    int top, const int* __restrict__ tile_group, const int* __restrict__ tile_row0,
                    const int* __restrict__ tile_rows, int M, int m_tiles, float limit, float alpha, float shift) {
    // the tile's activations, a stage of 64 k at a time, as 16-byte pieces [k piece][row]: a wave's operand
    // (16 rows of one piece) is 256 contiguous bytes
    __shared__ __attribute__((aligned(16))) hb_bf16x8 a_lds[2][GM_KSTEP / 8][MOE_TILE_M];
    int group, row0, rows;
    if (tile_group) {
        group = tile_group[blockIdx.y];
        if (group < 0) return;
        row0 = tile_row0[blockIdx.y];
        rows = tile_rows[blockIdx.y];
    } else {
        group = blockIdx.y / m_tiles;
        row0 = (blockIdx.y % m_tiles) * MOE_TILE_M;
        rows = M - row0 < MOE_TILE_M ? M - row0 : MOE_TILE_M;
    }
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;
    const int F = N / 2;
    const int out_cols = EPI == 2 ? F : N;
    // the wave's output columns: 64 of them, or with EPI 2 32 (from 32 gate rows and the 32 up rows that go with them)
    const int n0 = EPI == 2 ? (blockIdx.x * 4 + wave) * 32 : (blockIdx.x * 4 + wave) * 64;
    const bool idle = n0 >= out_cols;            // (such a wave still helps to load the activations)
    // W[g] lies in the operands' order [K / 32][N / 16][64 lanes][8]: a block of 16 rows and 32 k is 1 KB in a row
    const bf16* Wg = W + (size_t)group * N * K;
    const size_t kstep = (size_t)(N / 16) * 512;         // from a block to the same rows' next 32 k
    const bf16* wrow[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        int nb = (EPI == 2 ? (a < 2 ? n0 + 16 * a : F + n0 + 16 * (a - 2)) : n0 + 16 * a) / 16;
        if (nb >= N / 16 || idle) nb = N / 16 - 1;       // (read a block that exists; its sums are not stored)
        wrow[a] = Wg + (size_t)nb * 512 + lane * 8;
    }
    const int blocks = (rows + 15) / 16;
    // what this thread brings of a stage: rows tid / 8 and 32 + tid / 8, piece tid % 8
    const bf16* asrc[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        int m = 32 * j + tid / 8;
        if (m >= rows) m = rows - 1;
        const int src = top > 0 ? order[row0 + m] / top : row0 + m;
        asrc[j] = A + (size_t)src * lda + (size_t)group * a_group_off + (tid % 8) * 8;
    }
    hb_f32x4 acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = hb_f32x4{0.f, 0.f, 0.f, 0.f};

    const int stages = (K + GM_KSTEP - 1) / GM_KSTEP;
    hb_bf16x8 areg[2], wnext[2][4];
    auto fetch = [&](int st) {
        const int k0 = st * GM_KSTEP;
        const bool tail = k0 + (tid % 8) * 8 >= K;          // (K in steps of 32: the last stage may be half)
#pragma unroll
        for (int j = 0; j < 2; ++j) areg[j] = tail ? hb_bf16x8{} : *(const hb_bf16x8*)(asrc[j] + k0);
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int a = 0; a < 4; ++a)
                wnext[h][a] = k0 + 32 * h < K ? *(const hb_bf16x8*)(wrow[a] + (size_t)(k0 / 32 + h) * kstep) : hb_bf16x8{};
    };
    fetch(0);
    for (int st = 0; st < stages; ++st) {
        const int buf = st & 1;
#pragma unroll
        for (int j = 0; j < 2; ++j) a_lds[buf][tid % 8][32 * j + tid / 8] = areg[j];
        hb_bf16x8 wv[2][4];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int a = 0; a < 4; ++a) wv[h][a] = wnext[h][a];
        __syncthreads();          // the stage is in LDS (and the stage before the last has been read by all)
        if (st + 1 < stages) fetch(st + 1);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            hb_bf16x8 xv[4];
#pragma unroll
            for (int b = 0; b < 4; ++b)
                if (b < blocks) xv[b] = a_lds[buf][4 * h + g4][16 * b + r16];
#pragma unroll
            for (int b = 0; b < 4; ++b)
                if (b < blocks) {
#pragma unroll
                    for (int a = 0; a < 4; ++a)
                        acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[h][a], xv[b], acc[a][b], 0, 0, 0);
                }
        }
    }
    if (idle) return;
    // lane: activation row b * 16 + r16, weight rows g4 * 4 + i of each block
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const int m = b * 16 + r16;
        if (b >= blocks || m >= rows) continue;
        const size_t base = (size_t)(row0 + m) * ldc + (size_t)group * c_group_off;
        if (EPI == 2) {
            bf16* C = (bf16*)Cv;
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int n = n0 + 16 * a + g4 * 4 + i;
                    if (n >= F) continue;
                    const float g = fminf(acc[a][b][i], limit);
                    const float u = fminf(fmaxf(acc[a + 2][b][i], -limit), limit);
                    C[base + n] = hb_from_float<bf16>(g / (1.0f + expf(-alpha * g)) * (u + shift));
                }
        } else {
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int n = n0 + 16 * a + g4 * 4 + i;
                    if (n >= N) continue;
                    if (EPI == 0)
                        ((float*)Cv)[base + n] = acc[a][b][i];
                    else
                        ((bf16*)Cv)[base + n] = hb_from_float<bf16>(acc[a][b][i]);
                }
        }
    }
}

// The same for tiles of few rows (decoding): no stage in LDS and no barrier, a wave holds two blocks
// of weight rows, so that more waves stream the weights; every operand straight from memory.
template <int EPI>
__global__ void __launch_bounds__(256)
grouped_mfma_stream_kernel(const bf16* __restrict__ A, int lda, size_t a_group_off, const bf16* __restrict__ W, int N,
                    int K, void* __restrict__ Cv, int ldc, size_t c_group_off, const int* __restrict__ order,
                    int top, const int* __restrict__ tile_group, const int* __restrict__ tile_row0,
                    const int* __restrict__ tile_rows, int M, int m_tiles, float limit, float alpha, float shift) {
    int group, row0, rows;
    if (tile_group) {
        group = tile_group[blockIdx.y];
        if (group < 0) return;
        row0 = tile_row0[blockIdx.y];
        rows = tile_rows[blockIdx.y];
    } else {
        group = blockIdx.y / m_tiles;
        row0 = (blockIdx.y % m_tiles) * MOE_TILE_M;
        rows = M - row0 < MOE_TILE_M ? M - row0 : MOE_TILE_M;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g4 = lane >> 4;
    const int F = N / 2;
    const int out_cols = EPI == 2 ? F : N;
    // the first of the wave's output columns; its weight rows: [n0, n0 + 32), or with EPI 2 [n0, + 16) and [F + n0, + 16)
    const int n0 = EPI == 2 ? (blockIdx.x * 4 + wave) * 16 : (blockIdx.x * 4 + wave) * 32;
    if (n0 >= out_cols) return;
    const bf16* Wg = W + (size_t)group * N * K;
    const size_t kstep = (size_t)(N / 16) * 512;
    const bf16* wrow[2];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
        int nb = (EPI == 2 ? (a == 0 ? n0 : F + n0) : n0 + 16 * a) / 16;
        if (nb >= N / 16) nb = N / 16 - 1;           // (read a block that exists; its sums are not stored)
        wrow[a] = Wg + (size_t)nb * 512 + lane * 8;
    }
    const int blocks = (rows + 15) / 16;
    const bf16* xrow[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        int m = b * 16 + r16;
        if (m >= rows) m = rows - 1;
        const int src = top > 0 ? order[row0 + m] / top : row0 + m;
        xrow[b] = A + (size_t)src * lda + (size_t)group * a_group_off + g4 * 8;
    }
    hb_f32x4 acc[2][4];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = hb_f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll 4
    for (int k = 0; k < K; k += 32) {
        hb_bf16x8 wv[2], xv[4];
#pragma unroll
        for (int a = 0; a < 2; ++a) wv[a] = *(const hb_bf16x8*)(wrow[a] + (size_t)(k / 32) * kstep);
#pragma unroll
        for (int b = 0; b < 4; ++b)
            if (b < blocks) xv[b] = *(const hb_bf16x8*)(xrow[b] + k);
#pragma unroll
        for (int b = 0; b < 4; ++b)
            if (b < blocks) {
#pragma unroll
                for (int a = 0; a < 2; ++a)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[a], xv[b], acc[a][b], 0, 0, 0);
            }
    }
    // lane: activation row b * 16 + r16, weight rows g4 * 4 + i of each block
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const int m = b * 16 + r16;
        if (b >= blocks || m >= rows) continue;
        const size_t base = (size_t)(row0 + m) * ldc + (size_t)group * c_group_off;
        if (EPI == 2) {
            bf16* C = (bf16*)Cv;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int n = n0 + g4 * 4 + i;
                if (n >= F) continue;
                const float g = fminf(acc[0][b][i], limit);
                const float u = fminf(fmaxf(acc[1][b][i], -limit), limit);
                C[base + n] = hb_from_float<bf16>(g / (1.0f + expf(-alpha * g)) * (u + shift));
            }
        } else {
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int n = n0 + 16 * a + g4 * 4 + i;
                    if (n >= N) continue;
                    if (EPI == 0)
                        ((float*)Cv)[base + n] = acc[a][b][i];
                    else
                        ((bf16*)Cv)[base + n] = hb_from_float<bf16>(acc[a][b][i]);
                }
        }
    }
}

// tile_group null: `groups` groups of ceil(M / 64) tiles each over the same M rows; else a list of
// n_tiles tiles (a group < 0 ends a tile at once). K in steps of 32; lda, a_group_off and the matrices
// such that every operand's 8 numbers lie at a multiple of 16 bytes.
extern "C" int hb_grouped_mfma(const void* A, int lda, size_t a_group_off, const void* W, int N, int K, void* C,
                               int ldc, size_t c_group_off, int epi, const int* order, int top,
                               const int* tile_group, const int* tile_row0, const int* tile_rows, int n_tiles, int M,
                               int groups, float limit, float alpha, float shift, int few_rows, hipStream_t stream) {
    HB_REQUIRE(N > 0 && K > 0 && K % 32 == 0, "grouped product: K = %d must be a positive multiple of 32", K);
    HB_REQUIRE(N % 16 == 0 && (epi != 2 || N % 32 == 0), "grouped product: %d weight rows are no whole blocks of 16", N);
    HB_REQUIRE(lda % 8 == 0 && a_group_off % 8 == 0 && ((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0,
               "grouped product: operands must lie at multiples of 16 bytes");
    HB_REQUIRE(epi >= 0 && epi <= 2 && (epi != 2 || N % 2 == 0), "grouped product: unknown epilogue %d", epi);
    int m_tiles = 0, tiles = n_tiles;
    if (!tile_group) {
        HB_REQUIRE(M > 0 && groups > 0 && top == 0, "grouped product: empty batch");
        m_tiles = (M + MOE_TILE_M - 1) / MOE_TILE_M;
        tiles = m_tiles * groups;
    }
    HB_REQUIRE(tiles > 0 && tiles <= 65535, "grouped product: %d row tiles exceed the grid", tiles);
    const int out_cols = epi == 2 ? N / 2 : N;
    // few_rows: the tiles hold few rows each (the host knows how many rows there are to how many groups)
    const int per_group = few_rows ? (epi == 2 ? 64 : 128) : (epi == 2 ? 128 : 256);
    const dim3 grid((out_cols + per_group - 1) / per_group, tiles);
#define HB_GROUPED_STREAM(E)                                                                                        \
    grouped_mfma_stream_kernel<E><<<grid, 256, 0, stream>>>((const bf16*)A, lda, a_group_off, (const bf16*)W, N, K, \
                                                            C, ldc, c_group_off, order, top, tile_group, tile_row0,  \
                                                            tile_rows, M, m_tiles, limit, alpha, shift)
    if (few_rows) {
        if (epi == 0) HB_GROUPED_STREAM(0);
        else if (epi == 1) HB_GROUPED_STREAM(1);
        else HB_GROUPED_STREAM(2);
        HB_CHECK_LAUNCH("grouped_mfma_stream");
        return 0;
    }
#undef HB_GROUPED_STREAM
#define HB_GROUPED(E)                                                                                               \
    grouped_mfma_kernel<E><<<grid, 256, 0, stream>>>((const bf16*)A, lda, a_group_off, (const bf16*)W, N, K, C, ldc, \
                                                     c_group_off, order, top, tile_group, tile_row0, tile_rows, M,   \
                                                     m_tiles, limit, alpha, shift)
    if (epi == 0) HB_GROUPED(0);
    else if (epi == 1) HB_GROUPED(1);
    else HB_GROUPED(2);
#undef HB_GROUPED
    HB_CHECK_LAUNCH("grouped_mfma");
    return 0;
}
