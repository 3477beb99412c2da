// Kernels of mixers that carry a state of fixed size from token to token instead of keys and
// values: a filter of a few taps along time, channel by channel (its last inputs are state), and the
// gated delta rule, a matrix of state a head that every token first decays, then corrects towards
// its value along its key, then reads with its query. Everything here is float32.
//
// A step's tokens are packed over its sequences: row t belongs to sequence seq_of[t], whose rows
// are [seq_starts[i], seq_starts[i + 1]) and whose state lies at slot slots[i].
#include "common.h"
#include <math.h>

HB_MODULE_ERROR_SLOT()

#define HB_MAX_TAPS 16

__device__ __forceinline__ float hb_silu(float z) { return z / (1.0f + expf(-z)); }

// ------------------------------------------- convolution + silu (+ unit vectors a head)
// Channels are the first C columns of the projection's rows, in sections:
//   [n_unit sections of unit_dim channels | plain sections of plain_dim channels]
// y[t, c] = silu(sum_j taps[c, j] * in[t - (K - 1) + j, c]), the inputs before the step's first row
// from the slot's state [K - 1, C] (zeros in a fresh slot). A unit section is then divided by
// sqrt(sum of squares + unit_eps); sections below n_scaled are also multiplied by `scale`. With bias [C] the
// sum starts at bias[c]. The last plain section may be shorter than plain_dim (it ends with the channels).
// One wave a (token, section).
__global__ void __launch_bounds__(HB_WAVE)
conv_silu_kernel(const float* __restrict__ proj, int ld, const float* __restrict__ taps,
                 const float* __restrict__ conv_state, const int* __restrict__ seq_of,
                 const int* __restrict__ seq_starts, const int* __restrict__ slots, float* __restrict__ out,
                 int C, int K, int n_unit, int unit_dim, int n_scaled, float scale, float unit_eps,
                 int plain_dim, const float* __restrict__ bias) {
    const int t = blockIdx.x;
    const int sec = blockIdx.y;
    const int lane = threadIdx.x;
    const bool unit = sec < n_unit;
    const int c0 = unit ? sec * unit_dim : n_unit * unit_dim + (sec - n_unit) * plain_dim;
    const int len = unit ? unit_dim : (plain_dim < C - c0 ? plain_dim : C - c0);
    const int seq = seq_of[t];
    const int first = seq_starts[seq];
    const int at = t - first;                     // the token's place among the step's tokens of its sequence
    const float* state = conv_state + (size_t)slots[seq] * (K - 1) * C;
    float* row = out + (size_t)t * C;
    float ss = 0.f;
    for (int d = lane; d < len; d += HB_WAVE) {
        const int c = c0 + d;
        float acc = bias ? bias[c] : 0.f;
        for (int j = 0; j < K; ++j) {
            const int s = at - (K - 1) + j;
            const float v = s >= 0 ? proj[(size_t)(first + s) * ld + c] : state[(size_t)(K - 1 + s) * C + c];
            acc = fmaf(taps[(size_t)c * K + j], v, acc);
        }
        const float y = hb_silu(acc);
        row[c] = y;
        ss = fmaf(y, y, ss);
    }
    if (!unit) return;
    ss = hb_wave_sum(ss);
    const float inv = (sec < n_scaled ? scale : 1.0f) / sqrtf(ss + unit_eps);
    for (int d = lane; d < len; d += HB_WAVE) row[c0 + d] *= inv;     // (each lane rescales what it wrote)
}

// The state after the step: the last K - 1 inputs of each sequence, from the step's rows where it
// brought that many, else the old state moved up. One thread a (sequence, channel).
// (bias [C] or null: the inputs are the rows plus a bias a channel, and the state holds them with it)
__global__ void conv_state_kernel(const float* __restrict__ proj, int ld, float* __restrict__ conv_state,
                                  const int* __restrict__ seq_starts, const int* __restrict__ slots, int C,
                                  int K, const float* __restrict__ bias) {
    const int seq = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int first = seq_starts[seq], n = seq_starts[seq + 1] - first;
    float* state = conv_state + (size_t)slots[seq] * (K - 1) * C;
    const float b = bias ? bias[c] : 0.f;
    float keep[HB_MAX_TAPS];
    for (int i = 0; i < K - 1; ++i) {
        const int s = n - (K - 1) + i;
        keep[i] = s >= 0 ? proj[(size_t)(first + s) * ld + c] + b : state[(size_t)(i + n) * C + c];
    }
    for (int i = 0; i < K - 1; ++i) state[(size_t)i * C + c] = keep[i];
}

extern "C" int hb_conv_silu(const float* proj, int ld, const float* taps, float* conv_state, const int* seq_of,
                            const int* seq_starts, const int* slots, float* out, int T, int B, int C, int K,
                            int n_unit, int unit_dim, int n_scaled, float scale, float unit_eps, int n_plain,
                            int plain_dim, const float* bias, hipStream_t stream) {
    HB_REQUIRE(T > 0 && B > 0 && C > 0, "conv: empty input");
    HB_REQUIRE(K >= 1 && K <= HB_MAX_TAPS, "conv: %d taps, the kernel takes 1 to %d", K, HB_MAX_TAPS);
    HB_REQUIRE(n_unit * unit_dim + n_plain * plain_dim >= C && (n_plain == 0 ? n_unit * unit_dim == C
               : n_unit * unit_dim + (n_plain - 1) * plain_dim < C) && ld >= C,
               "conv: the sections do not add up to %d channels", C);
    HB_REQUIRE(n_unit + n_plain <= 65535 && B <= 65535, "conv: too many sections or sequences for the grid");
    conv_silu_kernel<<<dim3(T, n_unit + n_plain), HB_WAVE, 0, stream>>>(
        proj, ld, taps, conv_state, seq_of, seq_starts, slots, out, C, K, n_unit, unit_dim, n_scaled, scale,
        unit_eps, plain_dim, bias);
    HB_CHECK_LAUNCH("conv_silu");
    if (K > 1) {
        conv_state_kernel<<<dim3(B, (C + 255) / 256), 256, 0, stream>>>(proj, ld, conv_state, seq_starts, slots, C, K, nullptr);
        HB_CHECK_LAUNCH("conv_state");
    }
    return 0;
}

// The state of a filter alone, for mixers that filter in a kernel of their own: after a step, the last K - 1
// inputs (the first C columns of proj's rows, plus bias [C] if given) of each sequence.
extern "C" int hb_filter_state(const float* proj, int ld, float* conv_state, const int* seq_starts, const int* slots,
                               int B, int C, int K, const float* bias, hipStream_t stream) {
    HB_REQUIRE(B > 0 && C > 0 && ld >= C && B <= 65535, "filter state: empty input or too many sequences");
    HB_REQUIRE(K >= 1 && K <= HB_MAX_TAPS, "filter state: %d taps, the kernel takes 1 to %d", K, HB_MAX_TAPS);
    if (K == 1) return 0;
    conv_state_kernel<<<dim3(B, (C + 255) / 256), 256, 0, stream>>>(proj, ld, conv_state, seq_starts, slots, C, K, bias);
    HB_CHECK_LAUNCH("filter_state");
    return 0;
}

// ------------------------------------------------------------------ real-gated linear recurrent unit
// Two branches of W channels from one projection's rows [x | y] (float32, ld apart):
//   u[t, c] = fb[c] + sum_j taps[c, j] * (x[t - (K - 1) + j, c] + bx[c])     (nothing before a sequence's start; the
//             inputs before the step's first row come from the slot's state [K - 1, W], which holds them with bx)
//   g[t, c] = gelu_tanh(y[t, c] + by[c])
// out rows are [u | g], float32. One thread a (token, channel).
__device__ __forceinline__ float lru_gelu_tanh(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

__global__ void lru_inputs_kernel(const float* __restrict__ proj, int ld, const float* __restrict__ bx,
                                  const float* __restrict__ by, const float* __restrict__ taps,
                                  const float* __restrict__ fb, float* __restrict__ conv_state,
                                  const int* __restrict__ seq_of, const int* __restrict__ seq_starts,
                                  const int* __restrict__ slots, float* __restrict__ out, int W, int K,
                                  int moves_state) {
    const int t = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= W) return;
    const int seq = seq_of[t];
    const int first = seq_starts[seq];
    const int at = t - first;
    float* state = conv_state + (size_t)slots[seq] * (K > 1 ? K - 1 : 1) * W;
    const float b = bx[c];
    float acc = fb ? fb[c] : 0.f;
    if (moves_state) {
        // one token a sequence: this thread is the only reader of its channel's K - 1 kept inputs, so it also
        // moves them on (each takes the next one's place, the last the token's own input)
        for (int j = 0; j < K; ++j) {
            const float v = j < K - 1 ? state[(size_t)j * W + c] : proj[(size_t)t * ld + c] + b;
            acc = fmaf(taps[(size_t)c * K + j], v, acc);
            if (j > 0) state[(size_t)(j - 1) * W + c] = v;
        }
    } else {
        for (int j = 0; j < K; ++j) {
            const int s = at - (K - 1) + j;
            const float v = s >= 0 ? proj[(size_t)(first + s) * ld + c] + b : state[(size_t)(K - 1 + s) * W + c];
            acc = fmaf(taps[(size_t)c * K + j], v, acc);
        }
    }
    out[(size_t)t * 2 * W + c] = acc;
    out[(size_t)t * 2 * W + W + c] = lru_gelu_tanh(proj[(size_t)t * ld + W + c] + by[c]);
}

extern "C" int hb_lru_inputs(const float* proj, int ld, const float* bx, const float* by, const float* taps,
                             const float* fb, float* conv_state, const int* seq_of, const int* seq_starts,
                             const int* slots, float* out, int T, int B, int W, int K, int longest, hipStream_t stream) {
    HB_REQUIRE(T > 0 && B > 0 && W > 0 && ld >= 2 * W, "recurrent unit: empty input or rows of %d for 2 x %d channels", ld, W);
    HB_REQUIRE(K >= 1 && K <= HB_MAX_TAPS, "recurrent unit: %d taps, the kernel takes 1 to %d", K, HB_MAX_TAPS);
    HB_REQUIRE((W + 255) / 256 <= 65535 && B <= 65535, "recurrent unit: too many channels or sequences for the grid");
    // one token a sequence at most (longest: the most that a sequence of the step brings): the kernel moves the state on itself
    const int moves_state = longest == 1 && K > 1;
    lru_inputs_kernel<<<dim3(T, (W + 255) / 256), 256, 0, stream>>>(proj, ld, bx, by, taps, fb, conv_state, seq_of,
                                                                    seq_starts, slots, out, W, K, moves_state);
    HB_CHECK_LAUNCH("lru_inputs");
    if (K > 1 && !moves_state) {
        conv_state_kernel<<<dim3(B, (W + 255) / 256), 256, 0, stream>>>(proj, ld, conv_state, seq_starts, slots, W, K, bx);
        HB_CHECK_LAUNCH("lru_filter_state");
    }
    return 0;
}

// The recurrence itself, channel by channel:
//   r = sigmoid(r_pre[t, c] + rb[c]);  i = sigmoid(i_pre[t, c] + ib[c])
//       (gates rows are float32 [block 0: r, i | block 1: r, i | ...], blocks of bw channels, as a product a block
//        of the block's u with the block's two stacked matrices leaves them)
//   a = exp(-rate * r * softplus(lam[c]));  S <- a S + sqrt(1 - a^2) * i * u[t, c];  y[t, c] = S * g[t, c]
// with S from the slot's state [W] (zero in a fresh slot; the first token is no special case) and u, g the
// rows that lru_inputs_kernel left. 1 - a^2 is taken as -expm1(2 ln a), which keeps its digits where a is
// near one. One thread a (sequence, channel) walks the sequence's tokens; the loads of a token do not wait
// for the chain, which is one multiply-add long. Everything float32; y in any storage type.
template <class TOut>
__global__ void lru_scan_kernel(const float* __restrict__ ug, const float* __restrict__ gates,
                                const float* __restrict__ rb, const float* __restrict__ ib,
                                const float* __restrict__ lam, float rate, float* __restrict__ state,
                                const int* __restrict__ seq_starts, const int* __restrict__ slots,
                                TOut* __restrict__ y, int W, int bw) {
    const int seq = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= W) return;
    const int gc = (c / bw) * 2 * bw + c % bw;         // the channel's place among a row's gates
    const int first = seq_starts[seq], last = seq_starts[seq + 1];
    float* S_mem = state + (size_t)slots[seq] * W + c;
    float S = *S_mem;
    const float z = lam[c];
    const float step = -rate * (z > 20.f ? z : log1pf(expf(z)));
    const float rbc = rb[c], ibc = ib[c];
#pragma unroll 4
    for (int t = first; t < last; ++t) {
        const float r = 1.0f / (1.0f + expf(-(gates[(size_t)t * 2 * W + gc] + rbc)));
        const float i = 1.0f / (1.0f + expf(-(gates[(size_t)t * 2 * W + gc + bw] + ibc)));
        const float log_a = step * r;
        const float a = expf(log_a);
        const float in = sqrtf(-expm1f(2.0f * log_a)) * i * ug[(size_t)t * 2 * W + c];
        S = fmaf(a, S, in);
        y[(size_t)t * W + c] = hb_from_float<TOut>(S * ug[(size_t)t * 2 * W + W + c]);
    }
    *S_mem = S;
}

// The same recurrence for long portions, in two kernels. The first, one thread a (token, channel), turns the gates'
// pre-activations into the decay a and the input b = sqrt(1 - a^2) i u where they lie (`gates` is overwritten: r_pre's
// place takes a, i_pre's place b): the exponentials and the root are most of the arithmetic, and here they fill
// the chip. The second walks S_t = a_t S_(t-1) + b_t, a chain, but one whose pieces compose: over a run of tokens
// the state leaves as A S + B with A the product of the run's decays and B the run's walk from zero. A workgroup
// is SEGS waves on 64 channels; a sequence's tokens are cut into SEGS runs. Every wave but the last first walks
// its run from zero (A, B into LDS); then each wave takes the sequence's state through the runs before its own (at
// most SEGS - 1 multiply-adds) and walks its run again from there, now storing the outputs. The chain is two runs
// long instead of the whole portion. The result differs from the one-wave walk by float32 rounding (the runs' edges).
__global__ void lru_decay_input_kernel(const float* __restrict__ ug, float* __restrict__ gates,
                                       const float* __restrict__ rb, const float* __restrict__ ib,
                                       const float* __restrict__ lam, float rate, int W, int bw, size_t total) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const size_t t = idx / W;
    const int c = (int)(idx - t * W);
    const int gc = (c / bw) * 2 * bw + c % bw;
    float* row = gates + t * 2 * W;
    const float z = lam[c];
    const float step = -rate * (z > 20.f ? z : log1pf(expf(z)));
    const float r = 1.0f / (1.0f + expf(-(row[gc] + rb[c])));
    const float i = 1.0f / (1.0f + expf(-(row[gc + bw] + ib[c])));
    const float log_a = step * r;
    row[gc] = expf(log_a);
    row[gc + bw] = sqrtf(-expm1f(2.0f * log_a)) * i * ug[t * 2 * W + c];
}

template <class TOut, int SEGS>
__global__ void __launch_bounds__(64 * SEGS)
lru_scan_runs_kernel(const float* __restrict__ ug, const float* __restrict__ ab, float* __restrict__ state,
                     const int* __restrict__ seq_starts, const int* __restrict__ slots, TOut* __restrict__ y, int W, int bw) {
    __shared__ float sA[SEGS][64], sB[SEGS][64];
    const int seq = blockIdx.x;
    const int lane = threadIdx.x & 63, seg = threadIdx.x >> 6;
    const int c = blockIdx.y * 64 + lane;
    const bool live = c < W;
    const int cc = live ? c : 0;
    const int gc = (cc / bw) * 2 * bw + cc % bw;
    const int first = seq_starts[seq], n = seq_starts[seq + 1] - first;
    const int per = (n + SEGS - 1) / SEGS;
    const int t0 = first + min(seg * per, n), t1 = first + min((seg + 1) * per, n);
    float A = 1.f, B = 0.f;
    if (live && seg < SEGS - 1) {
#pragma unroll 8
        for (int t = t0; t < t1; ++t) {
            const float a = ab[(size_t)t * 2 * W + gc], in = ab[(size_t)t * 2 * W + gc + bw];
            B = fmaf(a, B, in);
            A *= a;
        }
    }
    sA[seg][lane] = A;
    sB[seg][lane] = B;
    __syncthreads();
    float* S_mem = state + (size_t)slots[seq] * W + cc;
    float S = live ? *S_mem : 0.f;
    for (int k = 0; k < seg; ++k) S = fmaf(sA[k][lane], S, sB[k][lane]);
    if (!live) return;
#pragma unroll 8
    for (int t = t0; t < t1; ++t) {
        const float a = ab[(size_t)t * 2 * W + gc], in = ab[(size_t)t * 2 * W + gc + bw];
        S = fmaf(a, S, in);
        y[(size_t)t * W + c] = hb_from_float<TOut>(S * ug[(size_t)t * 2 * W + W + c]);
    }
    if (seg == SEGS - 1) *S_mem = S;
}

// longest: the most tokens that one sequence of the step brings (the host knows it); portions of LRU_RUNS_FROM
// tokens or more take the kernel that cuts them into runs.
#define LRU_RUNS_FROM 128
#define LRU_RUNS 16

extern "C" int hb_lru_scan(const float* ug, float* gates, const float* rb, const float* ib, const float* lam,
                           float rate, float* state, const int* seq_starts, const int* slots, void* y, int y_dtype,
                           int B, int T, int W, int bw, int longest, hipStream_t stream) {
    HB_REQUIRE(B > 0 && W > 0 && B <= 65535, "recurrent unit: empty input or too many sequences for the grid");
    HB_REQUIRE(bw > 0 && W % bw == 0, "recurrent unit: %d channels in blocks of %d", W, bw);
    if (longest >= LRU_RUNS_FROM) {
        const size_t total = (size_t)T * W;
        HB_REQUIRE(T > 0 && (total + 255) / 256 <= 0x7fffffffu, "recurrent unit: %d tokens of %d channels exceed the grid", T, W);
        lru_decay_input_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(ug, gates, rb, ib, lam, rate, W, bw, total);
        HB_CHECK_LAUNCH("lru_decay_input");
        const dim3 grid(B, (W + 63) / 64);
        if (y_dtype == HB_F32)
            lru_scan_runs_kernel<float, LRU_RUNS><<<grid, 64 * LRU_RUNS, 0, stream>>>(ug, gates, state, seq_starts, slots, (float*)y, W, bw);
        else if (y_dtype == HB_BF16)
            lru_scan_runs_kernel<bf16, LRU_RUNS><<<grid, 64 * LRU_RUNS, 0, stream>>>(ug, gates, state, seq_starts, slots, (bf16*)y, W, bw);
        else
            HB_REQUIRE(false, "recurrent unit: unknown output dtype %d", y_dtype);
        HB_CHECK_LAUNCH("lru_scan_runs");
        return 0;
    }
    const int threads = W >= 4096 ? 256 : 64;          // (few channels: more, smaller workgroups over the CUs)
    const dim3 grid(B, (W + threads - 1) / threads);
    if (y_dtype == HB_F32)
        lru_scan_kernel<float><<<grid, threads, 0, stream>>>(ug, gates, rb, ib, lam, rate, state, seq_starts, slots, (float*)y, W, bw);
    else if (y_dtype == HB_BF16)
        lru_scan_kernel<bf16><<<grid, threads, 0, stream>>>(ug, gates, rb, ib, lam, rate, state, seq_starts, slots, (bf16*)y, W, bw);
    else
        HB_REQUIRE(false, "recurrent unit: unknown output dtype %d", y_dtype);
    HB_CHECK_LAUNCH("lru_scan");
    return 0;
}

// ------------------------------------------------------------------ gated delta rule
// State S [D, V] a (slot, head). For every token of the sequence, in order:
//   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q        (o sees the token's own write)
// with g = exp(-exp(A_log[h]) * softplus(a + dt_bias[h])) and beta = sigmoid(b), a and b columns of
// the projection's row. The columns of S never meet, and the tokens are a chain: the kernel is as
// fast as one token's step is short. A column is held by LPC lanes (each 8 or 16 of its D numbers, in
// registers; LPC = 1 .. 16 for D up to 256), a wave holds 64 / LPC columns and walks the sequence's
// tokens; a workgroup is one wave, so that a head's columns spread over many CUs. The two dot
// products a token are summed over a column's lanes by exchanges within a row of 16 lanes (the first
// runs on the numbers before their decay and is multiplied by g afterwards, g (S^T k) = (g S)^T k, so the
// decay itself does not wait for it). What a
// token needs (k, q, its values, g and beta, which do not wait for the chain) comes from a ring in
// LDS that is filled 16 to 32 tokens ahead: a token's own loads would each cost the memory's latency.
// qkv rows: [kv_heads x D queries | kv_heads x D keys | heads x V values]; head h reads the
// query and key of kv head h / (heads / kv_heads).
// Tokens that are loaded together, and such groups in the ring. A group's loads are issued before the
// group that is worked on and waited for after it, so a group must take longer than the memory's latency:
// with 8 tokens a group the kernel took that latency over 8 a token. (8 where 16 would not fit 64 KB of LDS.)
// CH: the decay is a factor a row of S (a key channel) instead of one a head: decay [T, heads x D] holds
// the factors themselves (hb_channel_decay makes them), and they come through the ring beside k and q.
// DELTA false (with CH): a linear attention with a decay a key channel, S <- diag(g) S + k v^T, o = S^T q: the same
// walk without the correction along the key (u = v) and without beta.
// C is what lies between two rows of qkv (at least the channels named above); o is multiplied by out_scale.
#define DELTA_SUB_OF(DP, CH) ((CH) ? ((DP) >= 128 ? 8 : 16) : ((DP) >= 256 ? 8 : 16))
#define DELTA_RING_OF(DP, CH) (((CH) && (DP) >= 256) ? 2 : 3)

__device__ __forceinline__ float delta_dpp(float v, const int ctrl) {
    // (a lane reads another lane's value: ctrl names which, within rows of 16 lanes)
    switch (ctrl) {
        case 0: return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));    // lane ^ 1
        case 1: return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));    // lane ^ 2
        case 2: return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));   // 7 - lane of each 8
        default: return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));  // 15 - lane of each 16
    }
}

// the sum over the LPC lanes of a column, in every one of them (after each step all lanes of a
// group of 2, 4, 8, 16 hold that group's sum, so a mirrored lane of the other half holds the other half's)
template <int LPC>
__device__ __forceinline__ float delta_column_sum(float v) {
    if (LPC >= 2) v += delta_dpp(v, 0);
    if (LPC >= 4) v += delta_dpp(v, 1);
    if (LPC >= 8) v += delta_dpp(v, 2);
    if (LPC >= 16) v += delta_dpp(v, 3);
    return v;
}

template <int LPC, int DELTA_PER, bool CH, bool DELTA>
__global__ void __launch_bounds__(HB_WAVE)
gated_delta_kernel(const float* __restrict__ qkv, int C, const float* __restrict__ proj, int ld, int b_off,
                   int a_off, const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                   const float* __restrict__ decay, float* __restrict__ state,
                   const int* __restrict__ seq_starts, const int* __restrict__ slots,
                   float* __restrict__ out, int kv_heads, int heads, int D, int V, float out_scale) {
    constexpr int COLS = HB_WAVE / LPC;
    constexpr int DP = LPC * DELTA_PER;                 // D rounded up to what the lanes hold
    constexpr int DELTA_RING = DELTA_RING_OF(DP, CH);
    constexpr int DELTA_SUB = DELTA_SUB_OF(DP, CH);
    constexpr int SLOTS = DELTA_SUB * DELTA_RING;
    constexpr int NB = CH ? 3 : 2;                      // blocks of DP numbers a token in the ring: k, q (, decay)
    constexpr int ROW4 = NB * DP / 4;                   // float4 of a token's ring row
    constexpr int KQ4 = DELTA_SUB * ROW4;               // float4 of k and q (and the decays) a group of tokens
    constexpr int KQ_PER_LANE = (KQ4 + HB_WAVE - 1) / HB_WAVE;
    constexpr int V_PER_LANE = (DELTA_SUB * COLS + HB_WAVE - 1) / HB_WAVE;
    __shared__ __attribute__((aligned(16))) float kq_ring[SLOTS][NB * DP];
    __shared__ float v_ring[SLOTS][COLS];
    __shared__ float gb_ring[SLOTS][2];
    const int seq = blockIdx.x, h = blockIdx.y;
    const int lane = threadIdx.x;
    const int part = lane % LPC;                       // which of the column's D numbers this lane holds
    const int lcol = lane / LPC;
    const int col0 = blockIdx.z * COLS;
    const int col = col0 + lcol;
    const bool live = col < V;
    const int d0 = part * DELTA_PER;
    const int kvh = h / (heads / kv_heads);
    const int first = seq_starts[seq], last = seq_starts[seq + 1];
    const int n_groups = (last - first + DELTA_SUB - 1) / DELTA_SUB;
    float* S_mem = state + ((size_t)slots[seq] * heads + h) * D * V + col;
    float S[DELTA_PER];
    // (numbers beyond D are zeros and stay zeros: their k and q are zeros in the ring)
#pragma unroll
    for (int i = 0; i < DELTA_PER; ++i) S[i] = (live && d0 + i < D) ? S_mem[(size_t)(d0 + i) * V] : 0.f;
    const float rate = CH ? 0.f : -expf(A_log[h]);
    const float bias = CH ? 0.f : dt_bias[h];
    const int g_ld = heads * D;
    const int q_at = kvh * D, k_at = (kv_heads + kvh) * D, v_at = 2 * kv_heads * D + h * V;
    const bool vec = (D % 4) == 0 && (C % 4) == 0;

    float4 kq_regs[KQ_PER_LANE];
    float v_regs[V_PER_LANE], g_reg = 0.f, beta_reg = 0.f;
    // group p of the sequence's tokens from memory into registers ...
    auto fetch = [&](int p) {
        const int t0 = first + p * DELTA_SUB;
#pragma unroll
        for (int j = 0; j < KQ_PER_LANE; ++j) {
            const int idx = j * HB_WAVE + lane;
            const int i = idx / ROW4, f = idx % ROW4;               // token of the group, float4 of its [k | q (| decay)]
            const int d = 4 * (f % (DP / 4));
            const int block = f / (DP / 4);
            float4 r = float4{0.f, 0.f, 0.f, 0.f};
            if (idx < KQ4 && t0 + i < last) {
                const float* src = (CH && block == 2) ? decay + (size_t)(t0 + i) * g_ld + (size_t)h * D + d
                                                      : qkv + (size_t)(t0 + i) * C + (block == 0 ? k_at : q_at) + d;
                if (vec && d + 3 < D) {
                    r = *(const float4*)src;
                } else {
                    if (d < D) r.x = src[0];
                    if (d + 1 < D) r.y = src[1];
                    if (d + 2 < D) r.z = src[2];
                    if (d + 3 < D) r.w = src[3];
                }
            }
            kq_regs[j] = r;
        }
#pragma unroll
        for (int j = 0; j < V_PER_LANE; ++j) {
            const int idx = j * HB_WAVE + lane;
            const int i = idx / COLS, c = idx % COLS;
            v_regs[j] = (idx < DELTA_SUB * COLS && t0 + i < last && col0 + c < V)
                            ? qkv[(size_t)(t0 + i) * C + v_at + col0 + c] : 0.f;
        }
        if (lane < DELTA_SUB && t0 + lane < last) {
            if (!CH) {
                const float z = proj[(size_t)(t0 + lane) * ld + a_off + h] + bias;
                const float softplus = z > 20.f ? z : log1pf(expf(z));
                g_reg = expf(rate * softplus);
            }
            if (DELTA) beta_reg = 1.0f / (1.0f + expf(-proj[(size_t)(t0 + lane) * ld + b_off + h]));
        }
    };
    // ... and from the registers into the ring
    auto stash = [&](int p) {
        const int s0 = (p % DELTA_RING) * DELTA_SUB;
#pragma unroll
        for (int j = 0; j < KQ_PER_LANE; ++j) {
            const int idx = j * HB_WAVE + lane;
            if (idx < KQ4) *(float4*)&kq_ring[s0 + idx / ROW4][4 * (idx % ROW4)] = kq_regs[j];
        }
#pragma unroll
        for (int j = 0; j < V_PER_LANE; ++j) {
            const int idx = j * HB_WAVE + lane;
            if (idx < DELTA_SUB * COLS) v_ring[s0 + idx / COLS][idx % COLS] = v_regs[j];
        }
        if (lane < DELTA_SUB) {
            gb_ring[s0 + lane][0] = g_reg;
            gb_ring[s0 + lane][1] = beta_reg;
        }
    };
    for (int p = 0; p < DELTA_RING - 1 && p < n_groups; ++p) {
        fetch(p);
        stash(p);
    }
    __syncthreads();
    for (int p = 0; p < n_groups; ++p) {
        const bool ahead = p + DELTA_RING - 1 < n_groups;
        if (ahead) fetch(p + DELTA_RING - 1);
        const int s0 = (p % DELTA_RING) * DELTA_SUB;
        const int t0 = first + p * DELTA_SUB;
        const int n = last - t0 < DELTA_SUB ? last - t0 : DELTA_SUB;
        for (int i = 0; i < n; ++i) {
            float kc[DELTA_PER], qc[DELTA_PER];
#pragma unroll
            for (int e = 0; e < DELTA_PER; e += 4) {
                const float4 kk = *(const float4*)&kq_ring[s0 + i][d0 + e];
                const float4 qq = *(const float4*)&kq_ring[s0 + i][DP + d0 + e];
                kc[e] = kk.x, kc[e + 1] = kk.y, kc[e + 2] = kk.z, kc[e + 3] = kk.w;
                qc[e] = qq.x, qc[e + 1] = qq.y, qc[e + 2] = qq.z, qc[e + 3] = qq.w;
            }
            const float vc = v_ring[s0 + i][lcol];
            const float g = gb_ring[s0 + i][0], beta = gb_ring[s0 + i][1];
            if (CH) {
                // a factor a row: the numbers decay first, then both dot products run on them
                float d4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int e = 0; e < DELTA_PER; e += 4) {
                    const float4 gg = *(const float4*)&kq_ring[s0 + i][2 * DP + d0 + e];
                    S[e] *= gg.x, S[e + 1] *= gg.y, S[e + 2] *= gg.z, S[e + 3] *= gg.w;
                }
                float u = vc;
                if (DELTA) {
#pragma unroll
                    for (int e = 0; e < DELTA_PER; ++e) d4[e & 3] = fmaf(S[e], kc[e], d4[e & 3]);
                    const float dot = delta_column_sum<LPC>((d4[0] + d4[1]) + (d4[2] + d4[3]));
                    u = beta * (vc - dot);
                }
                float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int e = 0; e < DELTA_PER; ++e) {
                    S[e] = fmaf(kc[e], u, S[e]);
                    o4[e & 3] = fmaf(S[e], qc[e], o4[e & 3]);
                }
                const float o = delta_column_sum<LPC>((o4[0] + o4[1]) + (o4[2] + o4[3]));
                if (live && part == 0) out[(size_t)(t0 + i) * heads * V + h * V + col] = o * out_scale;
                continue;
            }
            // g (S^T k) = (g S)^T k: the dot product runs on the old numbers, in four partial sums, and the
            // decay of the numbers themselves does not wait for it
            float d4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int e = 0; e < DELTA_PER; ++e) d4[e & 3] = fmaf(S[e], kc[e], d4[e & 3]);
            const float dot = g * delta_column_sum<LPC>((d4[0] + d4[1]) + (d4[2] + d4[3]));
            const float u = beta * (vc - dot);
            float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int e = 0; e < DELTA_PER; ++e) {
                S[e] = fmaf(kc[e], u, g * S[e]);
                o4[e & 3] = fmaf(S[e], qc[e], o4[e & 3]);
            }
            const float o = delta_column_sum<LPC>((o4[0] + o4[1]) + (o4[2] + o4[3]));
            if (live && part == 0) out[(size_t)(t0 + i) * heads * V + h * V + col] = o * out_scale;
        }
        if (ahead) stash(p + DELTA_RING - 1);           // (the place of the group before this one)
        __syncthreads();
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < DELTA_PER; ++i)
            if (d0 + i < D) S_mem[(size_t)(d0 + i) * V] = S[i];
    }
}

// decay null: one factor a head, from the projection's column a_off + h, A_log and dt_bias.
// decay [T, heads x D]: a factor a key channel, as given (a_off, A_log and dt_bias are not read).
// correction 0 (a decay a key channel must be given): the linear attention, S <- diag(g) S + k v^T; proj is not read.
extern "C" int hb_gated_delta(const float* qkv, int C, const float* proj, int ld, int b_off, int a_off,
                              const float* A_log, const float* dt_bias, const float* decay, float* state,
                              const int* seq_starts,
                              const int* slots, float* out, int B, int kv_heads, int heads, int D, int V,
                              int correction, float out_scale, hipStream_t stream) {
    HB_REQUIRE(correction || decay, "linear attention: the walk without a correction takes a decay a key channel");
    HB_REQUIRE(B > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "delta rule: %d heads on %d key heads", heads, kv_heads);
    HB_REQUIRE(D > 0 && D <= 256, "delta rule: keys of %d, the kernel takes 1 to 256", D);
    HB_REQUIRE(V > 0 && C >= 2 * kv_heads * D + heads * V, "delta rule: rows of %d do not hold the heads' channels", C);
    HB_REQUIRE(B <= 65535 && heads <= 65535, "delta rule: too many sequences or heads for the grid");
    // Lanes a column x numbers a lane. Few waves (one prompt of a model of up to 16 heads of 128 columns): 8 numbers a lane, so that a token's step is
    // short (the chain is what counts: 2,048 tokens of 16 heads of 128 x 128 take 0.97 ms with 16 numbers a
    // lane and 0.77 ms with 8). Many waves (a batch): 16 numbers a lane, half the waves and fewer
    // instructions in all (a decode step of 8 sequences: 15 us against 30).
    const int narrow = D <= 16 ? 1 : D <= 32 ? 2 : D <= 64 ? 4 : D <= 128 ? 8 : 16;        // lanes a column with 16 numbers a lane
    const long long waves = (long long)B * heads * ((V + HB_WAVE / narrow - 1) / (HB_WAVE / narrow));
    const bool wide = D <= 128 && (D <= 8 || waves <= 256);        // (twice as many must still run at once: three a CU by their LDS)
    const int lpc = wide ? (D <= 8 ? 1 : D <= 16 ? 2 : D <= 32 ? 4 : D <= 64 ? 8 : 16) : narrow;
    const int cols = HB_WAVE / lpc;
    const dim3 grid(B, heads, (V + cols - 1) / cols);
#define HB_DELTA(L, P)                                                                                            \
    do {                                                                                                          \
        if (decay && !correction)                                                                                 \
            gated_delta_kernel<L, P, true, false><<<grid, HB_WAVE, 0, stream>>>(qkv, C, proj, ld, b_off, a_off, A_log, \
                dt_bias, decay, state, seq_starts, slots, out, kv_heads, heads, D, V, out_scale);                 \
        else if (decay)                                                                                           \
            gated_delta_kernel<L, P, true, true><<<grid, HB_WAVE, 0, stream>>>(qkv, C, proj, ld, b_off, a_off, A_log, \
                dt_bias, decay, state, seq_starts, slots, out, kv_heads, heads, D, V, out_scale);                 \
        else                                                                                                      \
            gated_delta_kernel<L, P, false, true><<<grid, HB_WAVE, 0, stream>>>(qkv, C, proj, ld, b_off, a_off, A_log, \
                dt_bias, decay, state, seq_starts, slots, out, kv_heads, heads, D, V, out_scale);                 \
    } while (0)
    if (wide) {
        if (lpc == 1) HB_DELTA(1, 8);
        else if (lpc == 2) HB_DELTA(2, 8);
        else if (lpc == 4) HB_DELTA(4, 8);
        else if (lpc == 8) HB_DELTA(8, 8);
        else HB_DELTA(16, 8);
    } else {
        if (lpc == 1) HB_DELTA(1, 16);
        else if (lpc == 2) HB_DELTA(2, 16);
        else if (lpc == 4) HB_DELTA(4, 16);
        else if (lpc == 8) HB_DELTA(8, 16);
        else HB_DELTA(16, 16);
    }
#undef HB_DELTA
    HB_CHECK_LAUNCH("gated_delta");
    return 0;
}

// ------------------------------------- norm a head, weight, gate: what leaves the recurrence
// y[t, h, :] = o / sqrt(mean(o^2) + eps) * w * silu(gate[t, h, :]) (or sigmoid(gate), if so asked); w [V] is shared by the heads,
// the gate's pre-activations are columns [g_off + h V, ...) of the projection's row. One wave a (token, head).
template <class TOut>
__global__ void __launch_bounds__(HB_WAVE)
gated_head_norm_kernel(const float* __restrict__ o, const float* __restrict__ proj, int ld, int g_off,
                       const float* __restrict__ w, TOut* __restrict__ y, int heads, int V, float eps,
                       int sigmoid_gate) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* in = o + ((size_t)t * heads + h) * V;
    const float* gate = proj + (size_t)t * ld + g_off + (size_t)h * V;
    TOut* out = y + ((size_t)t * heads + h) * V;
    float ss = 0.f;
    for (int d = lane; d < V; d += HB_WAVE) ss = fmaf(in[d], in[d], ss);
    ss = hb_wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)V + eps);
    for (int d = lane; d < V; d += HB_WAVE) {
        const float z = gate[d];
        const float open = sigmoid_gate ? 1.0f / (1.0f + expf(-z)) : hb_silu(z);
        out[d] = hb_from_float<TOut>(in[d] * inv * w[d] * open);
    }
}

extern "C" int hb_gated_head_norm(const float* o, const float* proj, int ld, int g_off, const float* w, void* y,
                                  int y_dtype, int T, int heads, int V, float eps, int sigmoid_gate,
                                  hipStream_t stream) {
    HB_REQUIRE(T > 0 && heads > 0 && V > 0 && heads <= 65535, "gated norm: empty input or too many heads");
    if (y_dtype == HB_F32)
        gated_head_norm_kernel<float><<<dim3(T, heads), HB_WAVE, 0, stream>>>(o, proj, ld, g_off, w, (float*)y, heads, V, eps, sigmoid_gate);
    else if (y_dtype == HB_BF16)
        gated_head_norm_kernel<bf16><<<dim3(T, heads), HB_WAVE, 0, stream>>>(o, proj, ld, g_off, w, (bf16*)y, heads, V, eps, sigmoid_gate);
    else
        HB_REQUIRE(false, "gated norm: unknown output dtype %d", y_dtype);
    HB_CHECK_LAUNCH("gated_head_norm");
    return 0;
}

// ------------------------------------------------- a decay a key channel from its pre-activation
// g[t, h, d] = exp(-exp(A_log[h]) * softplus(z[t, h, d] + dt_bias[h, d])), float32; z's rows are ld apart
// (g's are heads x D apart, and g may be z itself where ld is that).
__global__ void channel_decay_kernel(const float* z, int ld, const float* __restrict__ A_log,
                                     const float* __restrict__ dt_bias, float* g, int D, int HD, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const size_t t = i / HD;
        const int c = (int)(i - t * HD);
        const float a = z[t * ld + c] + dt_bias[c];
        const float softplus = a > 20.f ? a : log1pf(expf(a));
        g[i] = expf(-expf(A_log[c / D]) * softplus);
    }
}

extern "C" int hb_channel_decay(const float* z, int ld, const float* A_log, const float* dt_bias, float* g, int T,
                                int heads, int D, hipStream_t stream) {
    HB_REQUIRE(T > 0 && heads > 0 && D > 0 && ld >= heads * D, "channel decay: empty input");
    const size_t n = (size_t)T * heads * D;
    const size_t blocks = (n + 255) / 256;
    channel_decay_kernel<<<(unsigned)(blocks > 16384 ? 16384 : blocks), 256, 0, stream>>>(z, ld, A_log, dt_bias, g,
                                                                                           D, heads * D, n);
    HB_CHECK_LAUNCH("channel_decay");
    return 0;
}

// ------------------------------------------------- state-space layer with one decay a head
// A head h (on group h / (heads / groups) of B and C) keeps S [N, P], zero when its sequence starts, and for
// every token, with dt = softplus(dt_pre[h] + dt_bias[h]) and a = exp(-exp(A_log[h]) dt):
//     S <- a S + dt B x^T;   y = S^T C + D[h] x.
// u f32 [T, ldu]: a row's columns are [x: heads x P | B: groups x N | C: groups x N] (what the convolution
// left); dt_pre: column dt_off + h of proj's rows (f32, ld apart); y f32 [T, heads x P]. Everything is float32.
// The state is the kernel's own: f32 [slots, heads, tiles, 256, NR], every thread's NR numbers of a (slot, head,
// tile of columns) side by side, so that a step of single tokens streams it in and out in whole lines; rows
// from N on and columns from P on are zeros and stay zeros.
// A workgroup is four waves on (256 / LPC columns of S, head, sequence): a column's N numbers lie over LPC lanes
// (4, 8 or 16), lane j holding rows j NR .. (j + 1) NR - 1, so the sum over N is NR products a lane and a few
// exchanges, in one order whatever the step holds; the more lanes a column has, the more waves a step of one
// sequence has and the shorter each wave's chain of work a token. The tokens are a chain; their inputs come
// through LDS eight tokens at a time, loaded by all four waves together, and the next eight are asked for (into
// registers) before the eight at hand are walked, so the chain does not wait for memory.
#define SSM_TOKENS 8
template <int NR, int LPC>
__global__ void __launch_bounds__(256)
ssm_scan_kernel(const float* __restrict__ u, int ldu, const float* __restrict__ proj, int ld, int dt_off,
                const float* __restrict__ dt_bias, const float* __restrict__ A_log, const float* __restrict__ Dskip,
                float* __restrict__ state, const int* __restrict__ seq_starts, const int* __restrict__ slots,
                float* __restrict__ y, int heads, int groups, int N, int P) {
    constexpr int CPW = 256 / LPC;                      // columns a workgroup
    constexpr int MAXN = LPC * NR;                      // rows that the lanes' registers hold (those from N on stay zero)
    constexpr int ROW = 2 * MAXN + CPW;                 // a token's inputs: B | C | x
    constexpr int STRIDE = ROW + 4;                     // then dt, the decay, and two unused
    constexpr int PER = (SSM_TOKENS * ROW + 255) / 256;
    __shared__ __attribute__((aligned(16))) float in_lds[SSM_TOKENS * STRIDE];
    const int tile = blockIdx.x, h = blockIdx.y, seq = blockIdx.z;
    const int tid = threadIdx.x, col = tid / LPC, part = tid % LPC;
    const int p = tile * CPW + col;
    const bool live = p < P;
    const int g = h / (heads / groups);
    const int first = seq_starts[seq], n_tok = seq_starts[seq + 1] - first;
    const int inner = heads * P;
    float* S = state + ((((size_t)slots[seq] * heads + h) * gridDim.x + tile) * 256 + tid) * NR;
    float s[NR];
#pragma unroll
    for (int i = 0; i < NR; i += 4) {
        const float4 held = *(const float4*)(S + i);
        s[i] = held.x, s[i + 1] = held.y, s[i + 2] = held.z, s[i + 3] = held.w;
    }
    const float rate = expf(A_log[h]), bias = dt_bias[h], skip = Dskip[h];
    // where this thread's PER numbers of a chunk lie in a token's row of u (below zero: nowhere; they are zeros)
    int src[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int idx = tid + 256 * i;
        const int e = idx % ROW;
        int off = -1;
        if (idx < SSM_TOKENS * ROW) {
            if (e < MAXN) off = e < N ? inner + g * N + e : -1;
            else if (e < 2 * MAXN) off = e - MAXN < N ? inner + (groups + g) * N + (e - MAXN) : -1;
            else off = tile * CPW + (e - 2 * MAXN) < P ? h * P + tile * CPW + (e - 2 * MAXN) : -1;
        }
        src[i] = off;
    }
    float pre[PER], pre_dt = 0.f;
    auto fetch = [&](int t0) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int k = (tid + 256 * i) / ROW;
            pre[i] = (src[i] >= 0 && t0 + k < n_tok) ? u[(size_t)(first + t0 + k) * ldu + src[i]] : 0.f;
        }
        pre_dt = (tid < SSM_TOKENS && t0 + tid < n_tok) ? proj[(size_t)(first + t0 + tid) * ld + dt_off + h] : 0.f;
    };
    fetch(0);
    for (int t0 = 0; t0 < n_tok; t0 += SSM_TOKENS) {
        const int nt = n_tok - t0 < SSM_TOKENS ? n_tok - t0 : SSM_TOKENS;
        __syncthreads();                 // (the chunk before has been walked)
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int idx = tid + 256 * i;
            if (idx < SSM_TOKENS * ROW) in_lds[(idx / ROW) * STRIDE + idx % ROW] = pre[i];
        }
        if (tid < SSM_TOKENS) {
            const float z = pre_dt + bias;
            const float dt = z > 20.f ? z : log1pf(expf(z));
            in_lds[tid * STRIDE + ROW] = dt;
            in_lds[tid * STRIDE + ROW + 1] = expf(-rate * dt);
        }
        __syncthreads();
        if (t0 + SSM_TOKENS < n_tok) fetch(t0 + SSM_TOKENS);
        for (int k = 0; k < nt; ++k) {
            const float* in = in_lds + k * STRIDE;
            const float x = in[2 * MAXN + col], dt = in[ROW], a = in[ROW + 1];
            const float dx = dt * x;
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < NR; i += 4) {
                const float4 b = *(const float4*)(in + part * NR + i);
                const float4 c = *(const float4*)(in + MAXN + part * NR + i);
                s[i] = fmaf(a, s[i], dx * b.x);
                s[i + 1] = fmaf(a, s[i + 1], dx * b.y);
                s[i + 2] = fmaf(a, s[i + 2], dx * b.z);
                s[i + 3] = fmaf(a, s[i + 3], dx * b.w);
                acc = fmaf(s[i], c.x, acc);
                acc = fmaf(s[i + 1], c.y, acc);
                acc = fmaf(s[i + 2], c.z, acc);
                acc = fmaf(s[i + 3], c.w, acc);
            }
#pragma unroll
            for (int off = 1; off < LPC; off <<= 1) acc += __shfl_xor(acc, off, HB_WAVE);
            if (live && part == 0) y[(size_t)(first + t0 + k) * inner + h * P + p] = fmaf(skip, x, acc);
        }
    }
#pragma unroll
    for (int i = 0; i < NR; i += 4) *(float4*)(S + i) = make_float4(s[i], s[i + 1], s[i + 2], s[i + 3]);
}

// How the kernel lays a head's state out: rows a lane (NR), lanes a column (LPC); 256 / LPC columns a tile.
static void ssm_layout(int N, int* nr, int* lpc) {
    if (N <= 16) *nr = 4, *lpc = 4;
    else if (N <= 32) *nr = 4, *lpc = 8;
    else if (N <= 64) *nr = 4, *lpc = 16;
    else if (N <= 128) *nr = 8, *lpc = 16;
    else *nr = 16, *lpc = 16;
}

// floats of state a (slot, head) for a state of N rows and P columns
extern "C" int hb_ssm_state_floats(int N, int P) {
    int nr, lpc;
    ssm_layout(N, &nr, &lpc);
    const int cpw = 256 / lpc;
    return (P + cpw - 1) / cpw * 256 * nr;
}

extern "C" int hb_ssm_scan(const float* u, int ldu, const float* proj, int ld, int dt_off, const float* dt_bias,
                           const float* A_log, const float* Dskip, float* state, const int* seq_starts,
                           const int* slots, float* y, int B, int heads, int groups, int N, int P,
                           int state_floats, hipStream_t stream) {
    HB_REQUIRE(B > 0 && heads > 0 && groups > 0 && N > 0 && P > 0, "state-space walk: empty input");
    HB_REQUIRE(N <= 256 && state_floats == hb_ssm_state_floats(N, P),
               "state-space walk: a head's state of %d floats is not the kernel's layout for %d x %d", state_floats, N, P);
    HB_REQUIRE(heads % groups == 0, "state-space walk: %d heads in %d groups", heads, groups);
    HB_REQUIRE(N <= 256, "state-space walk: a state of %d rows, the kernel takes up to 256", N);
    HB_REQUIRE(ldu >= heads * P + 2 * groups * N && dt_off >= 0 && dt_off + heads <= ld,
               "state-space walk: the columns lie outside their rows");
    HB_REQUIRE(heads <= 65535 && B <= 65535, "state-space walk: too many heads or sequences for the grid");
#define HB_SSM(NRV, LPCV)                                                                                              \
    ssm_scan_kernel<NRV, LPCV><<<dim3((P + 256 / LPCV - 1) / (256 / LPCV), heads, B), 256, 0, stream>>>(               \
        u, ldu, proj, ld, dt_off, dt_bias, A_log, Dskip, state, seq_starts, slots, y, heads, groups, N, P)
    int nr, lpc;
    ssm_layout(N, &nr, &lpc);
    if (nr == 4 && lpc == 4) HB_SSM(4, 4);
    else if (nr == 4 && lpc == 8) HB_SSM(4, 8);
    else if (nr == 4) HB_SSM(4, 16);
    else if (nr == 8) HB_SSM(8, 16);
    else HB_SSM(16, 16);
#undef HB_SSM
    HB_CHECK_LAUNCH("ssm_scan");
    return 0;
}

// ------------------------------------------------- gate, then a norm in groups: what leaves the state-space walk
// v = o silu(z); y = v / sqrt(mean over the group of v^2 + eps) * w: a row of `width` is cut into `parts` equal
// groups, each normed by its own root mean square; w [width]; z: columns [z_off, + width) of proj's rows.
// One workgroup a (token, group): a wave for groups of up to 256 channels, four waves beyond; the sum of squares
// runs in a fixed order.
template <class TOut>
__global__ void __launch_bounds__(256)
gated_group_norm_kernel(const float* __restrict__ o, const float* __restrict__ proj, int ld, int z_off,
                        const float* __restrict__ w, TOut* __restrict__ y, int width, int parts, float eps) {
    __shared__ float red[16];
    const int t = blockIdx.x, part = blockIdx.y, tid = threadIdx.x, nt = blockDim.x;
    const int len = width / parts, c0 = part * len;
    const float* in = o + (size_t)t * width + c0;
    const float* gate = proj + (size_t)t * ld + z_off + c0;
    float ss = 0.f;
    for (int d = tid; d < len; d += nt) {
        const float v = in[d] * hb_silu(gate[d]);
        ss = fmaf(v, v, ss);
    }
    ss = hb_block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)len + eps);
    for (int d = tid; d < len; d += nt)
        y[(size_t)t * width + c0 + d] = hb_from_float<TOut>(in[d] * hb_silu(gate[d]) * inv * w[c0 + d]);
}

extern "C" int hb_gated_group_norm(const float* o, const float* proj, int ld, int z_off, const float* w, void* y,
                                   int y_dtype, int T, int width, int parts, float eps, hipStream_t stream) {
    HB_REQUIRE(T > 0 && width > 0 && parts > 0 && width % parts == 0 && parts <= 65535,
               "gated norm in groups: %d columns in %d groups", width, parts);
    HB_REQUIRE(z_off >= 0 && z_off + width <= ld, "gated norm in groups: the gate's columns lie outside the rows");
    const int threads = width / parts > 256 ? 256 : HB_WAVE;
    if (y_dtype == HB_F32)
        gated_group_norm_kernel<float><<<dim3(T, parts), threads, 0, stream>>>(o, proj, ld, z_off, w, (float*)y, width, parts, eps);
    else if (y_dtype == HB_BF16)
        gated_group_norm_kernel<bf16><<<dim3(T, parts), threads, 0, stream>>>(o, proj, ld, z_off, w, (bf16*)y, width, parts, eps);
    else
        HB_REQUIRE(false, "gated norm in groups: unknown output dtype %d", y_dtype);
    HB_CHECK_LAUNCH("gated_group_norm");
    return 0;
}
