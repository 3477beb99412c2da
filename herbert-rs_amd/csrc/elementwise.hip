// Row-wise kernels of the decoder: embedding gather, RMSNorm, the fused
// per-head norm + rotation + cache write, and SwiGLU. All arithmetic is float32;
// the template parameters are the storage types of inputs and outputs.
// What each computes, in xigh/herbert-rs:
//   embedding        crates/backends/backend_common/src/generic_model.rs:104-111 (no multiplier; an id >= V is an error);
//                    crates/backends/backend_vulkan/shaders/embedding.comp:20-27
//   RMSNorm          crates/backends/backend_common/src/kernels.rs:54-64: x * 1 / sqrt(sum(x^2) / dim + eps) * w, eps inside
//                    the root, plain weight; crates/backends/backend_vulkan/shaders/rms_norm_batch.comp:25-41
//   per-head norm    crates/backends/backend_common/src/generic_attention/mod.rs:62-76 (before the rotation, the same eps,
//                    one weight [hd] for all heads, values untouched); backend_vulkan/shaders/head_rms_norm.comp:24-41
//   rotation         crates/backends/backend_common/src/kernels.rs:739-759 (pairs (j, j + R/2): x0 c - x1 s, x0 s + x1 c;
//                    elements from R on unchanged); tables crates/backends/backend_common/src/loader_common.rs:179-202
//   the three fused  crates/backends/backend_metal/shaders/head_norm_rope_kv_append.metal:37-110 (norm, rotation, append)
//   SwiGLU           crates/backends/backend_common/src/kernels.rs:676-687: g / (1 + exp(-g)) * u
#include "common.h"

HB_MODULE_ERROR_SLOT()

// ---------------------------------------------------------------- embedding
// x[t, :] = float(table[ids[t], :]); the residual stream is float32.
// PACKED: the table is stored in the MFMA kernels' order [H / 32][V / 16][64 lanes][8], element
// (n, k) at ((k / 32 * (V / 16) + n / 16) * 64 + (k / 8 % 4) * 16 + n % 16) * 8 + k % 8.
template <class TW, bool PACKED>
__global__ void embed_kernel(const int* __restrict__ ids, const TW* __restrict__ table,
                             float* __restrict__ x, int H, int V) {
    const int t = blockIdx.x;
    const int n = ids[t];
    float* out = x + (size_t)t * H;
    if ((unsigned)n >= (unsigned)V) {
        // The host checks the ids it sees; ids that come from the GPU (a sampler's output fed to the
        // next step) cannot be: a bad one reads nothing and makes its row NaN, which shows.
        for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = __uint_as_float(0x7fc00000u);
        return;
    }
    if (PACKED) {
        const TW* blk = table + (size_t)(n / 16) * 512 + (n % 16) * 8;
        const size_t plane = (size_t)(V / 16) * 512;
        for (int k = threadIdx.x; k < H; k += blockDim.x)
            out[k] = hb_to_float(blk[(size_t)(k / 32) * plane + ((k / 8) % 4) * 128 + (k % 8)]);
    } else {
        const TW* row = table + (size_t)n * H;
        if (sizeof(TW) == 2 && H % 8 == 0) {
            // eight bfloat16 a load (rows of a table whose width is a multiple of 8 start at 16 bytes)
            for (int i = threadIdx.x * 8; i < H; i += blockDim.x * 8) {
                const uint4 raw = *(const uint4*)(row + i);
                const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
                float v[8];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[2 * e] = __uint_as_float(w[e] << 16);
                    v[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
                }
                *(float4*)(out + i) = float4{v[0], v[1], v[2], v[3]};
                *(float4*)(out + i + 4) = float4{v[4], v[5], v[6], v[7]};
            }
            return;
        }
        for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = hb_to_float(row[i]);
    }
}

extern "C" int hb_embed(const int* ids, const void* table, int table_dtype, float* x, int T, int H, int V,
                        int packed, hipStream_t stream) {
    HB_REQUIRE(T > 0 && H > 0, "embed: empty input (T=%d, H=%d)", T, H);
    HB_REQUIRE(!packed || (table_dtype == HB_BF16 && H % 32 == 0 && V % 16 == 0),
               "embed: a packed table is bfloat16 with a width in steps of 32 and rows in steps of 16");
    if (table_dtype == HB_F32)
        embed_kernel<float, false><<<T, 256, 0, stream>>>(ids, (const float*)table, x, H, V);
    else if (table_dtype == HB_BF16 && packed)
        embed_kernel<bf16, true><<<T, 256, 0, stream>>>(ids, (const bf16*)table, x, H, V);
    else if (table_dtype == HB_BF16)
        embed_kernel<bf16, false><<<T, 256, 0, stream>>>(ids, (const bf16*)table, x, H, V);
    else
        HB_REQUIRE(false, "embed: unknown table dtype %d", table_dtype);
    HB_CHECK_LAUNCH("embed");
    return 0;
}

// ------------------------------------------------------------------ RMSNorm
// y[r, :] = x[src(r), :] * rsqrt(mean(x^2) + eps) * w ; src(r) = rows ? rows[r] : r.
// One block per output row; the sum's order depends on H and the block size only.
template <class TOut>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                               TOut* __restrict__ y, const int* __restrict__ rows, int H, float eps) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const float* in = x + (size_t)(rows ? rows[r] : r) * H;
    TOut* out = y + (size_t)r * H;
    float ss = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float v = in[i];
        ss += v * v;
    }
    ss = hb_block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
    for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = hb_from_float<TOut>(in[i] * inv * w[i]);
}

// The same for rows that fit the registers of one block (H in steps of 4, at most 8192): every
// element is loaded once, 16 bytes a lane, all loads in flight together.
typedef float hb_f4 __attribute__((ext_vector_type(4)));
// four neighbours of a row in one store (rows start at multiples of four elements)
__device__ __forceinline__ void store_four(float* out, hb_f4 v) { *(hb_f4*)out = v; }
__device__ __forceinline__ void store_four(bf16* out, hb_f4 v) {
    // (two conversions a register, round to nearest even as hb_from_float)
    typedef __bf16 hb_b2 __attribute__((ext_vector_type(2)));
    const hb_b2 lo = {(__bf16)v[0], (__bf16)v[1]}, hi = {(__bf16)v[2], (__bf16)v[3]};
    *(uint2*)out = uint2{__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi)};
}
template <class TOut>
__global__ void __launch_bounds__(256)
rmsnorm_row_kernel(const float* __restrict__ x, const float* __restrict__ w, TOut* __restrict__ y,
                   const int* __restrict__ rows, int H, float eps) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const hb_f4* in = (const hb_f4*)(x + (size_t)(rows ? rows[r] : r) * H);
    const hb_f4* w4 = (const hb_f4*)w;
    const int nv = H / 4;
    hb_f4 v[8], g[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const int i = threadIdx.x + 256 * c;
        if (i < nv) {
            v[c] = in[i];
            g[c] = w4[i];
        } else {
            v[c] = g[c] = hb_f4{0.f, 0.f, 0.f, 0.f};
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < 8; ++c) ss += v[c][0] * v[c][0] + v[c][1] * v[c][1] + v[c][2] * v[c][2] + v[c][3] * v[c][3];
    ss = hb_block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
    TOut* out = y + (size_t)r * H;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const int i = threadIdx.x + 256 * c;
        if (i < nv) {
            // (element by element: written as a product of vectors this took 380 registers)
            hb_f4 r;
#pragma unroll
            for (int e = 0; e < 4; ++e) r[e] = v[c][e] * inv * g[c][e];
            store_four(out + 4 * i, r);
        }
    }
}

extern "C" int hb_rmsnorm(const float* x, const float* w, void* y, int y_dtype, const int* rows, int R,
                          int H, float eps, hipStream_t stream) {
    HB_REQUIRE(R > 0 && H > 0, "rmsnorm: empty input (R=%d, H=%d)", R, H);
    HB_REQUIRE(y_dtype == HB_F32 || y_dtype == HB_BF16, "rmsnorm: unknown output dtype %d", y_dtype);
    if (H % 4 == 0 && H >= 1024 && H <= 8192) {
        if (y_dtype == HB_F32)
            rmsnorm_row_kernel<float><<<R, 256, 0, stream>>>(x, w, (float*)y, rows, H, eps);
        else
            rmsnorm_row_kernel<bf16><<<R, 256, 0, stream>>>(x, w, (bf16*)y, rows, H, eps);
    } else {
        const int threads = H >= 1024 ? 256 : 64;
        if (y_dtype == HB_F32)
            rmsnorm_kernel<float><<<R, threads, 0, stream>>>(x, w, (float*)y, rows, H, eps);
        else
            rmsnorm_kernel<bf16><<<R, threads, 0, stream>>>(x, w, (bf16*)y, rows, H, eps);
    }
    HB_CHECK_LAUNCH("rmsnorm");
    return 0;
}

// A query's factor at position p: 1 + coef * ln(floor((p + 1) / every) + 1); every <= 0: none.
__device__ __forceinline__ float hb_query_temperature(int pos, float coef, int every) {
    if (every <= 0) return 1.0f;
    return 1.0f + coef * logf((float)((pos + 1) / every) + 1.0f);
}

// ------------------------------------- per-head norm + rotation + cache write
// One wave per (token, head) of the fused projection row [q heads | k heads | v heads].
//   q heads: optional RMSNorm over the head, optional rotation, written to q_out.
//   k heads: the same, written to the key pages of the token's slot.
//   v heads: copied to the value pages, which are transposed: [page, kv head, hd, token].
// Rotation pairs dim j with j + R/2 (R = rot_dims), angle table [max_pos, R/2].
// The page of position p of a slot is page_table[slot * max_pages + p / page_size].
#define HB_MAX_HEAD_DIM 512

template <class TQ, class TC>
__global__ void qk_norm_rope_write_kernel(
    const float* __restrict__ qkv, int ld_qkv, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    int rot_dims, const int* __restrict__ positions, const int* __restrict__ seq_of,
    const int* __restrict__ slots, const int* __restrict__ page_table, int max_pages, int page_size,
    TQ* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache, int nq, int nkv, int hd,
    float eps, float q_temp_coef, int q_temp_every) {
    __shared__ float vec[HB_MAX_HEAD_DIM];
    const int t = blockIdx.x;
    const int h = blockIdx.y;
    const int lane = threadIdx.x;
    const float* src = qkv + (size_t)t * ld_qkv + (size_t)h * hd;
    const bool is_q = h < nq;
    const bool is_v = h >= nq + nkv;
    const int pos = positions[t];

    float ss = 0.f;
    for (int d = lane; d < hd; d += HB_WAVE) {
        const float v = src[d];
        vec[d] = v;
        ss += v * v;
    }
    ss = hb_wave_sum(ss);
    __syncthreads();

    const float* norm_w = is_q ? q_norm_w : k_norm_w;
    const bool do_norm = !is_v && norm_w != nullptr;
    const bool do_rope = !is_v && cos_t != nullptr;
    const float inv = do_norm ? 1.0f / sqrtf(ss / (float)hd + eps) : 1.0f;
    const int half = rot_dims / 2;
    // a query may grow with its position (see hb_query_temperature)
    const float grow = is_q ? hb_query_temperature(pos, q_temp_coef, q_temp_every) : 1.0f;

    size_t dst_base = 0;      // keys: start of the token's row; values: start of the (page, head) block
    if (!is_q) {
        const int slot = slots[seq_of[t]];
        const int page = page_table[(size_t)slot * max_pages + pos / page_size];
        const int kvh = is_v ? h - nq - nkv : h - nq;
        dst_base = ((size_t)page * nkv + kvh) * page_size * hd;
        if (!is_v) dst_base += (size_t)(pos % page_size) * hd;
    }
    const int in_page = pos % page_size;

    for (int d = lane; d < hd; d += HB_WAVE) {
        float out;
        if (do_rope && d < rot_dims) {
            const int j = d < half ? d : d - half;
            const float c = cos_t[(size_t)pos * half + j];
            const float s = sin_t[(size_t)pos * half + j];
            float x0 = vec[j], x1 = vec[j + half];
            if (do_norm) {
                x0 = x0 * inv * norm_w[j];
                x1 = x1 * inv * norm_w[j + half];
            }
            out = d < half ? x0 * c - x1 * s : x0 * s + x1 * c;
        } else {
            out = vec[d];
            if (do_norm) out = out * inv * norm_w[d];
        }
        if (is_q)
            q_out[(size_t)t * nq * hd + (size_t)h * hd + d] = hb_from_float<TQ>(out * grow);
        else if (is_v)
            v_cache[dst_base + (size_t)d * page_size + in_page] = hb_from_float<TC>(out);
        else
            k_cache[dst_base + d] = hb_from_float<TC>(out);
    }
}

// The same for many tokens (prompts), bfloat16 output, rotation over the whole head or none,
// head size in steps of 8 up to 128, rows of the projection 16-byte aligned: a workgroup takes 64
// consecutive tokens of one head. Query and key heads: half a wave a token, 16 bytes a lane.
// Value heads go through LDS, so that the transposed pages are written along the tokens: lane =
// token, 64 consecutive tokens of a page are one 128-byte line.
// QS > 1: the projection was cut into QS slices of K whose sums lie slice_stride floats apart
// behind qkv; they are added up in their order as they are loaded.
#define HB_TILED_HEAD_DIM 128
template <class TQ, class TC, int QS>
__global__ void __launch_bounds__(256) qk_norm_rope_write_tiled_kernel(
    const float* __restrict__ qkv, int ld_qkv, size_t slice_stride, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions, const int* __restrict__ seq_of, const int* __restrict__ slots,
    const int* __restrict__ page_table, int max_pages, int page_size, TQ* __restrict__ q_out,
    TC* __restrict__ k_cache, TC* __restrict__ v_cache, int T, int nq, int nkv, int hd, float eps,
    float q_temp_coef, int q_temp_every) {
    __shared__ float vt[64][HB_TILED_HEAD_DIM + 1];
    const int t0 = blockIdx.x * 64, h = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool is_q = h < nq, is_v = h >= nq + nkv;
    const int half = hd / 2;
    auto summed4 = [&](const float* p) {
        hb_f4 part[QS];
#pragma unroll
        for (int i = 0; i < QS; ++i) part[i] = *(const hb_f4*)(p + (size_t)i * slice_stride);
        hb_f4 sum = part[0];
#pragma unroll
        for (int i = 1; i < QS; ++i) sum += part[i];
        return sum;
    };
    if (is_v) {
        const int kvh = h - nq - nkv;
        const int q4 = hd / 4;                       // 16-byte chunks of a row
        for (int idx = tid; idx < 64 * q4; idx += 256) {
            const int r = idx / q4, c = (idx - r * q4) * 4;
            const int t = t0 + r;
            hb_f4 v = {0.f, 0.f, 0.f, 0.f};
            if (t < T) v = summed4(qkv + (size_t)t * ld_qkv + (size_t)h * hd + c);
#pragma unroll
            for (int e = 0; e < 4; ++e) vt[r][c + e] = v[e];
        }
        __syncthreads();
        const int t = t0 + lane;
        if (t >= T) return;
        const int pos = positions[t];
        const int page = page_table[(size_t)slots[seq_of[t]] * max_pages + pos / page_size];
        TC* dst = v_cache + ((size_t)page * nkv + kvh) * page_size * hd + pos % page_size;
        for (int d = wave; d < hd; d += 4) dst[(size_t)d * page_size] = hb_from_float<TC>(vt[lane][d]);
        return;
    }
    // Query and key heads: half a wave a token, a lane four consecutive elements (16 bytes in, 8
    // out); the lanes l < hd / 8 hold the first half of the head, their partners l + hd / 8 the
    // elements they are rotated with. A wave's 16 tokens go in two rounds of 8 (4 passes of 2
    // tokens): all loads of a round go out before anything waits for them.
    const float* norm_w = is_q ? q_norm_w : k_norm_w;
    const int l = lane & 31, sub = lane >> 5;
    const int eighth = hd / 8;
    const bool mine = l < 2 * eighth;
    const bool first = l < eighth;
    const int d0 = mine ? 4 * l : 0;
    const int j0 = mine && !first ? d0 - half : d0;              // where this lane's angles lie
    const int partner = (lane & 32) + (mine ? (first ? l + eighth : l - eighth) : l);
    hb_f4 w = {1.f, 1.f, 1.f, 1.f};
    if (norm_w && mine) w = *(const hb_f4*)(norm_w + d0);
#pragma unroll
    for (int round = 0; round < 2; ++round) {
        hb_f4 x[4], c[4], sn[4];
        int pos[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int t = t0 + 16 * wave + 8 * round + 2 * u + sub;
            const int tc = t < T ? t : T - 1;
            pos[u] = positions[tc];
            x[u] = hb_f4{0.f, 0.f, 0.f, 0.f};
            if (mine) x[u] = summed4(qkv + (size_t)tc * ld_qkv + (size_t)h * hd + d0);
        }
        if (cos_t) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                c[u] = *(const hb_f4*)(cos_t + (size_t)pos[u] * half + j0);
                sn[u] = *(const hb_f4*)(sin_t + (size_t)pos[u] * half + j0);
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int t = t0 + 16 * wave + 8 * round + 2 * u + sub;
            hb_f4 a = x[u];
            if (norm_w) {
                float ss = a[0] * a[0] + a[1] * a[1] + a[2] * a[2] + a[3] * a[3];
#pragma unroll
                for (int d = 1; d < 32; d <<= 1) ss += __shfl_xor(ss, d, 64);
                const float inv = 1.0f / sqrtf(ss / (float)hd + eps);
#pragma unroll
                for (int e = 0; e < 4; ++e) a[e] = a[e] * inv * w[e];
            }
            if (cos_t) {
                hb_f4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float other = __shfl(a[e], partner, 64);
                    // first half: x0 c - x1 s; second half: x0 s + x1 c (x0 the partner's element)
                    o[e] = first ? a[e] * c[u][e] - other * sn[u][e] : other * sn[u][e] + a[e] * c[u][e];
                }
                a = o;
            }
            if (!mine || t >= T) continue;
            if (is_q && q_temp_every > 0) {
                const float grow = hb_query_temperature(pos[u], q_temp_coef, q_temp_every);
#pragma unroll
                for (int e = 0; e < 4; ++e) a[e] *= grow;
            }
            TQ packed[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) packed[e] = hb_from_float<TQ>(a[e]);
            if (is_q) {
                *(uint2*)(q_out + ((size_t)t * nq + h) * hd + d0) = *(const uint2*)packed;
            } else {
                const int page = page_table[(size_t)slots[seq_of[t]] * max_pages + pos[u] / page_size];
                *(uint2*)(k_cache + (((size_t)page * nkv + (h - nq)) * page_size + pos[u] % page_size) * hd + d0) =
                    *(const uint2*)packed;
            }
        }
    }
}

extern "C" int hb_qk_norm_rope_write(const float* qkv, int ld_qkv, const float* q_norm_w,
                                     const float* k_norm_w, const float* cos_t, const float* sin_t,
                                     int rot_dims, const int* positions, const int* seq_of,
                                     const int* slots, const int* page_table, int max_pages,
                                     int page_size, void* q_out, void* k_cache, void* v_cache, int dtype,
                                     int T, int nq, int nkv, int hd, float eps, int write_kv,
                                     int qkv_slices, size_t slice_stride, float q_temp_coef, int q_temp_every,
                                     hipStream_t stream) {
    HB_REQUIRE(T > 0 && nq > 0 && nkv > 0, "qk_norm_rope_write: empty input");
    HB_REQUIRE(hd > 0 && hd <= HB_MAX_HEAD_DIM, "qk_norm_rope_write: head_dim %d not in 1..%d", hd,
               HB_MAX_HEAD_DIM);
    HB_REQUIRE(rot_dims % 2 == 0 && rot_dims >= 0 && rot_dims <= hd,
               "qk_norm_rope_write: rotary dims %d must be even and <= head_dim %d", rot_dims, hd);
    // write_kv == 0: the row holds query heads only and the cache is left alone
    const int heads = nq + (write_kv ? 2 * nkv : 0);
    HB_REQUIRE(ld_qkv >= heads * hd, "qk_norm_rope_write: row stride %d too small", ld_qkv);
    HB_REQUIRE(heads <= 65535, "qk_norm_rope_write: too many heads for the grid");
    if (dtype == HB_BF16 && write_kv && T >= 64 && hd <= HB_TILED_HEAD_DIM && hd % 8 == 0 && ld_qkv % 4 == 0 &&
        slice_stride % 4 == 0 && ((uintptr_t)qkv & 15) == 0 &&
        (cos_t == nullptr || rot_dims == hd) && (T + 63) / 64 <= 0x7fffffff) {
        dim3 tiles((T + 63) / 64, heads);
        HB_REQUIRE(qkv_slices == 1 || slice_stride >= (size_t)T * ld_qkv, "qk_norm_rope_write: slices overlap");
#define TILED_GO(QSV)                                                                                          \
    qk_norm_rope_write_tiled_kernel<bf16, bf16, QSV><<<tiles, 256, 0, stream>>>(                              \
        qkv, ld_qkv, slice_stride, q_norm_w, k_norm_w, cos_t, sin_t, positions, seq_of, slots, page_table,    \
        max_pages, page_size, (bf16*)q_out, (bf16*)k_cache, (bf16*)v_cache, T, nq, nkv, hd, eps, q_temp_coef,   \
        q_temp_every)
        if (qkv_slices == 1) TILED_GO(1);
        else if (qkv_slices == 2) TILED_GO(2);
        else if (qkv_slices == 4) TILED_GO(4);
        else if (qkv_slices == 8) TILED_GO(8);
        else HB_REQUIRE(false, "qk_norm_rope_write: %d slices of the projection are not taken", qkv_slices);
#undef TILED_GO
        HB_CHECK_LAUNCH("qk_norm_rope_write_tiled");
        return 0;
    }
    HB_REQUIRE(qkv_slices == 1, "qk_norm_rope_write: only the kernel for bfloat16 prompts of 64 tokens or more adds up slices");
    dim3 grid(T, heads);
    if (dtype == HB_F32)
        qk_norm_rope_write_kernel<float, float><<<grid, HB_WAVE, 0, stream>>>(
            qkv, ld_qkv, q_norm_w, k_norm_w, cos_t, sin_t, rot_dims, positions, seq_of, slots,
            page_table, max_pages, page_size, (float*)q_out, (float*)k_cache, (float*)v_cache, nq, nkv,
            hd, eps, q_temp_coef, q_temp_every);
    else if (dtype == HB_BF16)
        qk_norm_rope_write_kernel<bf16, bf16><<<grid, HB_WAVE, 0, stream>>>(
            qkv, ld_qkv, q_norm_w, k_norm_w, cos_t, sin_t, rot_dims, positions, seq_of, slots,
            page_table, max_pages, page_size, (bf16*)q_out, (bf16*)k_cache, (bf16*)v_cache, nq, nkv, hd,
            eps, q_temp_coef, q_temp_every);
    else
        HB_REQUIRE(false, "qk_norm_rope_write: unknown dtype %d", dtype);
    HB_CHECK_LAUNCH("qk_norm_rope_write");
    return 0;
}

// ------------------------------------------------------------------- gated linear units
// act[t, i] = f(gu[t, i]) * gu[t, I + i] with f = silu, g / (1 + exp(-g)), or the tanh form of gelu,
// 0.5 g (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3))).
#define HB_ACT_SILU 0
#define HB_ACT_GELU_TANH 1
__device__ __forceinline__ float hb_gelu_tanh(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <class TOut, int ACT>
__global__ void swiglu_kernel(const float* __restrict__ gu, TOut* __restrict__ act, int I, size_t total) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const size_t t = idx / I;
    const int i = (int)(idx - t * I);
    const float g = gu[t * 2 * I + i];
    const float u = gu[t * 2 * I + I + i];
    const float f = ACT == HB_ACT_GELU_TANH ? hb_gelu_tanh(g) : g / (1.0f + expf(-g));
    act[idx] = hb_from_float<TOut>(f * u);
}

extern "C" int hb_swiglu(const float* gu, void* act, int act_dtype, int T, int I, int activation, hipStream_t stream) {
    HB_REQUIRE(T > 0 && I > 0, "swiglu: empty input");
    HB_REQUIRE(activation == HB_ACT_SILU || activation == HB_ACT_GELU_TANH, "swiglu: unknown activation %d", activation);
    HB_REQUIRE(act_dtype == HB_F32 || act_dtype == HB_BF16, "swiglu: unknown output dtype %d", act_dtype);
    const size_t total = (size_t)T * I;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (act_dtype == HB_F32) {
        if (activation == HB_ACT_SILU) swiglu_kernel<float, HB_ACT_SILU><<<blocks, 256, 0, stream>>>(gu, (float*)act, I, total);
        else swiglu_kernel<float, HB_ACT_GELU_TANH><<<blocks, 256, 0, stream>>>(gu, (float*)act, I, total);
    } else {
        if (activation == HB_ACT_SILU) swiglu_kernel<bf16, HB_ACT_SILU><<<blocks, 256, 0, stream>>>(gu, (bf16*)act, I, total);
        else swiglu_kernel<bf16, HB_ACT_GELU_TANH><<<blocks, 256, 0, stream>>>(gu, (bf16*)act, I, total);
    }
    HB_CHECK_LAUNCH("swiglu");
    return 0;
}

// ------------------------------------------------------------------ fill
// A small fill kernel: clears memory inside captured graphs, where a memset node may not stand.
__global__ void fill_u32_kernel(uint32_t* p, uint32_t v, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

extern "C" int hb_fill_u32(void* p, uint32_t value, size_t n, hipStream_t stream) {
    if (n == 0) return 0;
    fill_u32_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>((uint32_t*)p, value, n);
    HB_CHECK_LAUNCH("fill_u32");
    return 0;
}

// ---------------------------------------------------------------- layer norm
// y[r, :] = (x[src(r), :] - mean) / sqrt(var + eps) * w, var = the mean of the squared deviations
// (two passes over the row: the deviations are taken from the mean, not from sums of squares);
// no bias. y may be x itself (float32, no gather): every element is read by the thread that writes it,
// and all reads of a pass are done before the block's sum is.
// DELTA: the row is first x + mult * delta (the sum of a layer's parts joins the residual stream),
// written back to x, and that sum is what is normed: one kernel between two layers.
template <class TOut, bool DELTA>
__global__ void layernorm_kernel(float* x, const float* __restrict__ delta, float mult,
                                 const float* __restrict__ w, TOut* y, const int* __restrict__ rows, int H,
                                 float eps) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const size_t src = (size_t)(rows ? rows[r] : r) * H;
    float* in = x + src;
    TOut* out = y + (size_t)r * H;
    float s = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        float v = in[i];
        if (DELTA) {
            v = fmaf(mult, delta[src + i], v);
            in[i] = v;
        }
        s += v;
    }
    const float mean = hb_block_sum(s, red) / (float)H;
    float ss = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float d = in[i] - mean;
        ss += d * d;
    }
    ss = hb_block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
    if (y == nullptr) return;
    for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = hb_from_float<TOut>((in[i] - mean) * inv * w[i]);
}

// delta may be null (a plain layer norm). With delta, rows must be null and x is updated in place;
// y null: only the sum is wanted (after the last layer).
extern "C" int hb_layernorm(float* x, const float* delta, float mult, const float* w, void* y, int y_dtype,
                            const int* rows, int R, int H, float eps, hipStream_t stream) {
    HB_REQUIRE(R > 0 && H > 0, "layernorm: empty input (R=%d, H=%d)", R, H);
    HB_REQUIRE(y_dtype == HB_F32 || y_dtype == HB_BF16, "layernorm: unknown output dtype %d", y_dtype);
    HB_REQUIRE(delta == nullptr || rows == nullptr, "layernorm: rows are not gathered while a sum is added");
    HB_REQUIRE(y != nullptr || delta != nullptr, "layernorm: nothing to do");
    const int threads = H >= 1024 ? 256 : H >= 256 ? 128 : 64;
    if (delta) {
        if (y_dtype == HB_F32)
            layernorm_kernel<float, true><<<R, threads, 0, stream>>>(x, delta, mult, w, (float*)y, rows, H, eps);
        else
            layernorm_kernel<bf16, true><<<R, threads, 0, stream>>>(x, delta, mult, w, (bf16*)y, rows, H, eps);
    } else {
        if (y_dtype == HB_F32)
            layernorm_kernel<float, false><<<R, threads, 0, stream>>>(x, nullptr, 0.f, w, (float*)y, rows, H, eps);
        else
            layernorm_kernel<bf16, false><<<R, threads, 0, stream>>>(x, nullptr, 0.f, w, (bf16*)y, rows, H, eps);
    }
    HB_CHECK_LAUNCH("layernorm");
    return 0;
}

// ---------------------------------------------------------------- x = x * s (float32, in place)
__global__ void scale_kernel(float* x, float s, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        x[i] *= s;
}

extern "C" int hb_scale(float* x, float s, size_t n, hipStream_t stream) {
    HB_REQUIRE(n > 0, "scale: empty input");
    const size_t blocks = (n + 255) / 256;
    scale_kernel<<<(unsigned)(blocks > 4096 ? 4096 : blocks), 256, 0, stream>>>(x, s, n);
    HB_CHECK_LAUNCH("scale");
    return 0;
}

// ------------------------------------------------- a layer whose norm comes after the sum
// Between two parts of such a layer the stream is x <- norm(alpha x + part(x)). The parts add their
// outputs to rows that already hold alpha x; this kernel then makes from such rows `src`, a row a block,
//   x = src / sqrt(mean(src^2) + eps) * w      (w null: x = src, the stream's first rows)
//   y = x in the compute dtype                 (what the next part reads; null: none)
//   acc = alpha_next x                         (where the next part adds; alpha_next 0: left alone)
// x may be null too (nobody reads the float32 rows). acc may be src itself (every element is read by
// the thread that writes it, after the row's sum is done); x and y are other rows than src.
template <class TOut>
__global__ void postnorm_kernel(const float* src, const float* __restrict__ w, float* __restrict__ x,
                                TOut* __restrict__ y, float* acc, int H, float eps, float alpha_next) {
    __shared__ float red[16];
    const size_t row = (size_t)blockIdx.x * H;
    float inv = 1.0f;
    if (w) {
        float ss = 0.f;
        for (int i = threadIdx.x; i < H; i += blockDim.x) {
            const float v = src[row + i];
            ss = fmaf(v, v, ss);
        }
        ss = hb_block_sum(ss, red);
        inv = 1.0f / sqrtf(ss / (float)H + eps);
    }
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float v = w ? src[row + i] * inv * w[i] : src[row + i];
        if (x) x[row + i] = v;
        if (y) y[row + i] = hb_from_float<TOut>(v);
        if (alpha_next != 0.f) acc[row + i] = alpha_next * v;
    }
}

// The same with a row's numbers kept in registers between the sum of squares and the writes (VPT float4 a
// thread): one read of src instead of two. H in steps of 4, at most 4 x VPT x blockDim.x; rows on 16-byte borders.
template <class TOut, int VPT>
__global__ void postnorm_held_kernel(const float* src, const float* __restrict__ w, float* __restrict__ x,
                                     TOut* __restrict__ y, float* acc, int H, float eps, float alpha_next) {
    __shared__ float red[16];
    const size_t row = (size_t)blockIdx.x * H;
    const int quads = H / 4;
    float4 v[VPT];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int q = threadIdx.x + j * blockDim.x;
        v[j] = q < quads ? *(const float4*)(src + row + 4 * q) : make_float4(0.f, 0.f, 0.f, 0.f);
        ss = fmaf(v[j].x, v[j].x, ss), ss = fmaf(v[j].y, v[j].y, ss);
        ss = fmaf(v[j].z, v[j].z, ss), ss = fmaf(v[j].w, v[j].w, ss);
    }
    float inv = 1.0f;
    if (w) {
        ss = hb_block_sum(ss, red);
        inv = 1.0f / sqrtf(ss / (float)H + eps);
    }
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        const int q = threadIdx.x + j * blockDim.x;
        if (q >= quads) continue;
        float4 o = v[j];
        if (w) {
            const float4 ww = *(const float4*)(w + 4 * q);
            o.x = o.x * inv * ww.x, o.y = o.y * inv * ww.y, o.z = o.z * inv * ww.z, o.w = o.w * inv * ww.w;
        }
        const size_t at = row + 4 * q;
        if (x) *(float4*)(x + at) = o;
        if (y) {
            y[at] = hb_from_float<TOut>(o.x), y[at + 1] = hb_from_float<TOut>(o.y);
            y[at + 2] = hb_from_float<TOut>(o.z), y[at + 3] = hb_from_float<TOut>(o.w);
        }
        if (alpha_next != 0.f)
            *(float4*)(acc + at) = make_float4(alpha_next * o.x, alpha_next * o.y, alpha_next * o.z, alpha_next * o.w);
    }
}

template <class TOut>
static bool postnorm_held(const float* src, const float* w, float* x, TOut* y, float* acc, int R, int H, float eps,
                          float alpha_next, int threads, hipStream_t stream) {
    const uintptr_t all = (uintptr_t)src | (uintptr_t)w | (uintptr_t)x | (uintptr_t)acc;
    if (H % 4 || all % 16) return false;
    const int per = (H / 4 + threads - 1) / threads;
#define HB_HELD(V) postnorm_held_kernel<TOut, V><<<R, threads, 0, stream>>>(src, w, x, y, acc, H, eps, alpha_next)
    if (per <= 1) HB_HELD(1);
    else if (per <= 2) HB_HELD(2);
    else if (per <= 4) HB_HELD(4);
    else if (per <= 8) HB_HELD(8);
    else return false;
#undef HB_HELD
    return true;
}

extern "C" int hb_postnorm(const float* src, const float* w, float* x, void* y, int y_dtype, float* acc, int R, int H,
                           float eps, float alpha_next, hipStream_t stream) {
    HB_REQUIRE(alpha_next == 0.f || acc != nullptr, "postnorm: no rows for alpha x");
    HB_REQUIRE(R > 0 && H > 0, "postnorm: empty input (R=%d, H=%d)", R, H);
    HB_REQUIRE(y_dtype == HB_F32 || y_dtype == HB_BF16, "postnorm: unknown output dtype %d", y_dtype);
    const int threads = H >= 2048 ? 256 : H >= 512 ? 128 : 64;
    if (y_dtype == HB_F32) {
        if (!postnorm_held<float>(src, w, x, (float*)y, acc, R, H, eps, alpha_next, threads, stream))
            postnorm_kernel<float><<<R, threads, 0, stream>>>(src, w, x, (float*)y, acc, H, eps, alpha_next);
    } else {
        if (!postnorm_held<bf16>(src, w, x, (bf16*)y, acc, R, H, eps, alpha_next, threads, stream))
            postnorm_kernel<bf16><<<R, threads, 0, stream>>>(src, w, x, (bf16*)y, acc, H, eps, alpha_next);
    }
    HB_CHECK_LAUNCH("postnorm");
    return 0;
}

// ---------------------------------------------------------------- squared relu
// act[i] = max(z[i], 0)^2, float32 in, any storage type out.
template <class TOut>
__global__ void relu_squared_kernel(const float* __restrict__ z, TOut* __restrict__ act, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const float r = fmaxf(z[i], 0.f);
        act[i] = hb_from_float<TOut>(r * r);
    }
}

extern "C" int hb_relu_squared(const float* z, void* act, int act_dtype, size_t n, hipStream_t stream) {
    HB_REQUIRE(n > 0, "relu_squared: empty input");
    const size_t blocks = (n + 255) / 256;
    const unsigned grid = (unsigned)(blocks > 16384 ? 16384 : blocks);
    if (act_dtype == HB_F32)
        relu_squared_kernel<float><<<grid, 256, 0, stream>>>(z, (float*)act, n);
    else if (act_dtype == HB_BF16)
        relu_squared_kernel<bf16><<<grid, 256, 0, stream>>>(z, (bf16*)act, n);
    else
        HB_REQUIRE(false, "relu_squared: unknown output dtype %d", act_dtype);
    HB_CHECK_LAUNCH("relu_squared");
    return 0;
}

// ------------------------------------------- RMSNorm that first takes a scaled sum on
// x[r, :] += ls * delta[r, :] (ls a factor a column), written back to x, then y[r, :] = x / rms(x) * w: the
// one kernel between two branches of a pre-norm layer whose branches are scaled channel by channel.
// y null: only the sum (after the last layer).
template <class TOut>
__global__ void rmsnorm_scaled_sum_kernel(float* x, const float* __restrict__ delta, const float* __restrict__ ls,
                                          const float* __restrict__ w, TOut* y, int H, float eps) {
    __shared__ float red[16];
    const size_t row = (size_t)blockIdx.x * H;
    float* in = x + row;
    float ss = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float v = fmaf(ls[i], delta[row + i], in[i]);
        in[i] = v;
        ss += v * v;
    }
    if (y == nullptr) return;
    ss = hb_block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
    TOut* out = y + row;
    for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = hb_from_float<TOut>(in[i] * inv * w[i]);
}

// The same for rows of up to 4096 numbers in steps of four: a thread keeps its up to sixteen sums in registers
// between the two passes (16-byte loads and stores), so that the second pass waits for no memory.
template <class TOut>
__global__ void __launch_bounds__(256)
rmsnorm_scaled_sum_held_kernel(float* x, const float* __restrict__ delta, const float* __restrict__ ls,
                               const float* __restrict__ w, TOut* y, int H, float eps) {
    __shared__ float red[16];
    const size_t row = (size_t)blockIdx.x * H;
    const int quads = H / 4;
    float4 held[4];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int q = threadIdx.x + j * 256;
        if (q < quads) {
            const float4 a = *(const float4*)(x + row + 4 * q), d = *(const float4*)(delta + row + 4 * q);
            const float4 f = *(const float4*)(ls + 4 * q);
            float4 v;
            v.x = fmaf(f.x, d.x, a.x), v.y = fmaf(f.y, d.y, a.y), v.z = fmaf(f.z, d.z, a.z), v.w = fmaf(f.w, d.w, a.w);
            *(float4*)(x + row + 4 * q) = v;
            held[j] = v;
            ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
    }
    if (y == nullptr) return;
    ss = hb_block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int q = threadIdx.x + j * 256;
        if (q < quads) {
            const float4 g = *(const float4*)(w + 4 * q);
            TOut* out = y + row + 4 * q;
            out[0] = hb_from_float<TOut>(held[j].x * inv * g.x);
            out[1] = hb_from_float<TOut>(held[j].y * inv * g.y);
            out[2] = hb_from_float<TOut>(held[j].z * inv * g.z);
            out[3] = hb_from_float<TOut>(held[j].w * inv * g.w);
        }
    }
}

extern "C" int hb_rmsnorm_scaled_sum(float* x, const float* delta, const float* ls, const float* w, void* y,
                                     int y_dtype, int R, int H, float eps, hipStream_t stream) {
    HB_REQUIRE(R > 0 && H > 0, "rmsnorm: empty input (R=%d, H=%d)", R, H);
    HB_REQUIRE(delta != nullptr && ls != nullptr, "rmsnorm: a scaled sum needs its rows and its factors");
    HB_REQUIRE(y == nullptr || w != nullptr, "rmsnorm: a norm needs its weight");
    HB_REQUIRE(y_dtype == HB_F32 || y_dtype == HB_BF16, "rmsnorm: unknown output dtype %d", y_dtype);
    if (H % 4 == 0 && H >= 1024 && H <= 4096 && (uintptr_t)x % 16 == 0 && (uintptr_t)delta % 16 == 0 &&
        (uintptr_t)ls % 16 == 0 && (w == nullptr || (uintptr_t)w % 16 == 0)) {
        if (y_dtype == HB_F32)
            rmsnorm_scaled_sum_held_kernel<float><<<R, 256, 0, stream>>>(x, delta, ls, w, (float*)y, H, eps);
        else
            rmsnorm_scaled_sum_held_kernel<bf16><<<R, 256, 0, stream>>>(x, delta, ls, w, (bf16*)y, H, eps);
        HB_CHECK_LAUNCH("rmsnorm_scaled_sum_held");
        return 0;
    }
    const int threads = H >= 1024 ? 256 : H >= 256 ? 128 : 64;
    if (y_dtype == HB_F32)
        rmsnorm_scaled_sum_kernel<float><<<R, threads, 0, stream>>>(x, delta, ls, w, (float*)y, H, eps);
    else
        rmsnorm_scaled_sum_kernel<bf16><<<R, threads, 0, stream>>>(x, delta, ls, w, (bf16*)y, H, eps);
    HB_CHECK_LAUNCH("rmsnorm_scaled_sum");
    return 0;
}

// ------------------------------------------- two rows normed and weighed into one
// out[r, :] (+)= ca * a[r, :] / rms(a[r]) * wa + cb * b[r, :] / rms(b[r]) * wb: the outputs of two mixers
// that ran side by side, each normed over the model's width, joined. float32 throughout.
template <bool ACCUM>
__global__ void normed_pair_kernel(const float* __restrict__ a, const float* __restrict__ wa, float ca,
                                   const float* __restrict__ b, const float* __restrict__ wb, float cb,
                                   float* out, int H, float eps) {
    __shared__ float red[16];
    const size_t row = (size_t)blockIdx.x * H;
    float sa = 0.f, sb = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float va = a[row + i], vb = b[row + i];
        sa += va * va;
        sb += vb * vb;
    }
    sa = hb_block_sum(sa, red);
    sb = hb_block_sum(sb, red);
    const float ia = ca / sqrtf(sa / (float)H + eps), ib = cb / sqrtf(sb / (float)H + eps);
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float v = a[row + i] * ia * wa[i] + b[row + i] * ib * wb[i];
        out[row + i] = ACCUM ? out[row + i] + v : v;
    }
}

// The same for rows of up to 4096 numbers in steps of four: both rows stay in registers between the two passes.
template <bool ACCUM>
__global__ void __launch_bounds__(256)
normed_pair_held_kernel(const float* __restrict__ a, const float* __restrict__ wa, float ca,
                        const float* __restrict__ b, const float* __restrict__ wb, float cb, float* out, int H, float eps) {
    __shared__ float red[16];
    const size_t row = (size_t)blockIdx.x * H;
    const int quads = H / 4;
    float4 ha[4], hb[4];
    float sa = 0.f, sb = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int q = threadIdx.x + j * 256;
        if (q < quads) {
            ha[j] = *(const float4*)(a + row + 4 * q);
            hb[j] = *(const float4*)(b + row + 4 * q);
            sa += ha[j].x * ha[j].x + ha[j].y * ha[j].y + ha[j].z * ha[j].z + ha[j].w * ha[j].w;
            sb += hb[j].x * hb[j].x + hb[j].y * hb[j].y + hb[j].z * hb[j].z + hb[j].w * hb[j].w;
        }
    }
    sa = hb_block_sum(sa, red);
    sb = hb_block_sum(sb, red);
    const float ia = ca / sqrtf(sa / (float)H + eps), ib = cb / sqrtf(sb / (float)H + eps);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int q = threadIdx.x + j * 256;
        if (q < quads) {
            const float4 ga = *(const float4*)(wa + 4 * q), gb = *(const float4*)(wb + 4 * q);
            float4 v;
            v.x = ha[j].x * ia * ga.x + hb[j].x * ib * gb.x;
            v.y = ha[j].y * ia * ga.y + hb[j].y * ib * gb.y;
            v.z = ha[j].z * ia * ga.z + hb[j].z * ib * gb.z;
            v.w = ha[j].w * ia * ga.w + hb[j].w * ib * gb.w;
            float4* o = (float4*)(out + row + 4 * q);
            if (ACCUM) {
                const float4 p = *o;
                v.x += p.x, v.y += p.y, v.z += p.z, v.w += p.w;
            }
            *o = v;
        }
    }
}

extern "C" int hb_normed_pair(const float* a, const float* wa, float ca, const float* b, const float* wb, float cb,
                              float* out, int R, int H, float eps, int accumulate, hipStream_t stream) {
    HB_REQUIRE(R > 0 && H > 0, "normed pair: empty input (R=%d, H=%d)", R, H);
    if (H % 4 == 0 && H >= 1024 && H <= 4096 &&
        (((uintptr_t)a | (uintptr_t)b | (uintptr_t)wa | (uintptr_t)wb | (uintptr_t)out) & 15) == 0) {
        if (accumulate)
            normed_pair_held_kernel<true><<<R, 256, 0, stream>>>(a, wa, ca, b, wb, cb, out, H, eps);
        else
            normed_pair_held_kernel<false><<<R, 256, 0, stream>>>(a, wa, ca, b, wb, cb, out, H, eps);
        HB_CHECK_LAUNCH("normed_pair_held");
        return 0;
    }
    const int threads = H >= 1024 ? 256 : H >= 256 ? 128 : 64;
    if (accumulate)
        normed_pair_kernel<true><<<R, threads, 0, stream>>>(a, wa, ca, b, wb, cb, out, H, eps);
    else
        normed_pair_kernel<false><<<R, threads, 0, stream>>>(a, wa, ca, b, wb, cb, out, H, eps);
    HB_CHECK_LAUNCH("normed_pair");
    return 0;
}

// ------------------------------------------- filter along time + norm over the whole projection
//                                             + rotation of neighbouring pairs + cache write
// A row of the fused projection holds [nq x dim queries | nkv x dim keys | nkv x vdim values] in its first
// C columns. One workgroup a token:
//   filter (taps [C, K], K >= 1; null: none): y[c] = sum_j taps[c, j] * in[t - (K - 1) + j, c], the inputs
//     before the step's first row from the slot's state [K - 1, C] (zeros in a fresh slot); the state is
//     moved on by a kernel of its own afterwards (hb_filter_state in the module of the recurrent mixers), or
//     here where every sequence brings one token;
//   bias (null: none): bias[c] is added to channel c after the filter;
//   norm (weights null: none): all queries of the token are divided by their common root mean square and
//     multiplied by q_norm_w [nq x dim], the keys likewise with k_norm_w [nkv x dim]; with head_norm every
//     query head and every key head is divided by its own root mean square instead, and the weights are
//     q_norm_w [dim] and k_norm_w [dim], the same for every head;
//   rotation (rates null: none): entries 2i and 2i + 1 of the first rot_dims of every query and key head turn
//     by position x rates[i]; rates and the angle are float64, sine and cosine float32 of the angle reduced to [-pi, pi];
//   q_out [T, nq x hd], key pages [page, kv head, token, hd], value pages [page, kv head, hd, token]: heads
//     are kept at size hd >= max(dim, vdim), the entries beyond a head's own size are zeros.
// TK: the taps' count where it is 2, 3 or 4 (the filter's loop is then unrolled and all of a thread's loads of an
// iteration are in flight together), 0: any count.
// NT: threads a token: a quarter of 1024 where the step has many tokens, 1024 where it has few (a token's
// channels are then spread over sixteen waves, which hide each other's waits).
template <class TQ, class TC, int TK, int NT>
__global__ void __launch_bounds__(NT)
filter_norm_rotate_write_kernel(const float* __restrict__ proj, int ld, const float* __restrict__ taps, int K,
                                float* __restrict__ filter_state, const float* __restrict__ q_norm_w,
                                const float* __restrict__ k_norm_w, const double* __restrict__ rates, int rot_dims,
                                const int* __restrict__ positions, const int* __restrict__ seq_of,
                                const int* __restrict__ seq_starts, const int* __restrict__ slots,
                                const int* __restrict__ page_table, int max_pages, int page_size,
                                TQ* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache, int nq,
                                int nkv, int dim, int vdim, int hd, float eps, int moves_state,
                                const float* __restrict__ bias, int head_norm) {
    constexpr int U = NT == 256 ? 8 : 4;          // channels a thread handles at a time
    extern __shared__ float filtered[];           // [C] the token's channels, then [rot_dims] cosines and sines, then [nq + nkv] a head's 1 / rms
    __shared__ float red[16];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int QD = nq * dim, KD = nkv * dim, C = QD + KD + nkv * vdim;
    float* cs = filtered + C;
    const int seq = seq_of[t];
    const int first = seq_starts[seq];
    const int at = t - first;
    const int slot = slots[seq];
    const int pos = positions[t];
    float* state = filter_state + (size_t)slot * (K > 1 ? K - 1 : 1) * C;
    const int page = page_table[(size_t)slot * max_pages + pos / page_size];       // (asked for early: used last)
    const int in_page = pos % page_size;
    // (the angles first: their loads then wait beside the filter's, not after them)
    if (rates != nullptr) {
        for (int i = tid; i < rot_dims / 2; i += NT) {
            // the angle and its reduction to [-pi, pi] in float64 (a few operations), sine and cosine of the reduced
            // angle in float32: a float64 sincos costs as much as the rest of the kernel
            const double a = (double)pos * rates[i];
            const double turns = rint(a * 0.15915494309189535);
            const double r = fma(-turns, 1.2246467991473532e-16 * 2.0, fma(-turns, 6.283185307179586, a));
            float s, c;
            sincosf((float)r, &s, &c);
            cs[2 * i] = c;
            cs[2 * i + 1] = s;
        }
    }
    float sq = 0.f, sk = 0.f;
    // U channels a thread at a time, so that a tap's U loads are in flight together (one channel after
    // the other, every load would wait for the one before: the taps' count is not known when this is compiled)
    for (int c0 = tid; c0 < C; c0 += U * NT) {
        float y[U], wn[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            // the norm's weight of the channel, loaded here beside the filter's operands: the loops that store the
            // heads then read LDS only and wait for no memory
            const int c = c0 + u * NT;
            y[u] = (bias != nullptr && c < C) ? bias[c] : 0.f;
            wn[u] = 1.f;
            if (head_norm) continue;                  // (a head's weights are applied where the heads are stored)
            if (c < QD) { if (q_norm_w) wn[u] = q_norm_w[c]; }
            else if (c < QD + KD) { if (k_norm_w) wn[u] = k_norm_w[c - QD]; }
        }
        if (taps == nullptr) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int c = c0 + u * NT;
                if (c < C) y[u] += proj[(size_t)t * ld + c];
            }
        } else {
            if (TK > 0) {
                // the taps' count is known: every load of the eight channels is asked for before anything is stored
                // (a store into the state would hold back the loads behind it, which may read the state)
                constexpr int N = TK > 0 ? TK : 1;
                float v[N][U], w[N][U];
#pragma unroll
                for (int j = 0; j < N; ++j) {
                    const int s = at - (N - 1) + j;
                    const float* row = s >= 0 ? proj + (size_t)(first + s) * ld : state + (size_t)(N - 1 + s) * C;
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const int c = c0 + u * NT;
                        v[j][u] = c < C ? row[c] : 0.f;
                        w[j][u] = c < C ? taps[(size_t)c * N + j] : 0.f;
                    }
                }
#pragma unroll
                for (int j = 0; j < N; ++j)
#pragma unroll
                    for (int u = 0; u < U; ++u) y[u] = fmaf(w[j][u], v[j][u], y[u]);
                // one token a sequence: this thread is the only reader of its channels' kept inputs and moves
                // them on itself (each takes the place of the one before it, the last the token's own input)
                if (moves_state) {
#pragma unroll
                    for (int j = 1; j < N; ++j)
#pragma unroll
                        for (int u = 0; u < U; ++u) {
                            const int c = c0 + u * NT;
                            if (c < C) state[(size_t)(j - 1) * C + c] = v[j][u];
                        }
                }
            } else {
                for (int j = 0; j < K; ++j) {
                    const int s = at - (K - 1) + j;
                    const float* row = s >= 0 ? proj + (size_t)(first + s) * ld : state + (size_t)(K - 1 + s) * C;
                    float v[U], w[U];
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const int c = c0 + u * NT;
                        v[u] = c < C ? row[c] : 0.f;
                        w[u] = c < C ? taps[(size_t)c * K + j] : 0.f;
                    }
#pragma unroll
                    for (int u = 0; u < U; ++u) y[u] = fmaf(w[u], v[u], y[u]);
                    if (moves_state && j > 0) {
#pragma unroll
                        for (int u = 0; u < U; ++u) {
                            const int c = c0 + u * NT;
                            if (c < C) state[(size_t)(j - 1) * C + c] = v[u];
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int c = c0 + u * NT;
            if (c >= C) continue;
            filtered[c] = y[u] * wn[u];
            if (c < QD) sq = fmaf(y[u], y[u], sq);
            else if (c < QD + KD) sk = fmaf(y[u], y[u], sk);
        }
    }
    sq = hb_block_sum(sq, red);           // (its barriers also publish `filtered` and the angles)
    sk = hb_block_sum(sk, red);
    const float inv_q = q_norm_w ? 1.0f / sqrtf(sq / (float)QD + eps) : 1.0f;
    const float inv_k = k_norm_w ? 1.0f / sqrtf(sk / (float)KD + eps) : 1.0f;
    const int rd = rates != nullptr ? rot_dims : 0;
    float* const inv_head = cs + rd;
    if (head_norm) {
        // a wave a head: its sum of squares in one order whatever else the step holds
        const int lane = tid & 63;
        for (int h = tid >> 6; h < nq + nkv; h += NT / 64) {
            float ss = 0.f;
            for (int d = lane; d < dim; d += 64) ss = fmaf(filtered[h * dim + d], filtered[h * dim + d], ss);
            ss = hb_wave_sum(ss);
            if (lane == 0) inv_head[h] = 1.0f / sqrtf(ss / (float)dim + eps);
        }
        __syncthreads();
    }
    // one entry of a query or key head after norm and rotation; c0: the head's first channel
    auto turned = [&](int c0, int d, float inv) {
        if (d >= dim) return 0.f;
        const float* const hw = !head_norm ? nullptr : c0 < QD ? q_norm_w : k_norm_w;
        if (head_norm) inv = inv_head[c0 / dim];
        // (without head_norm the weight is in `filtered` already)
        auto normed = [&](int e) { return filtered[c0 + e] * inv * (hw ? hw[e] : 1.0f); };
        if (d >= rd) return normed(d);
        const int i = d >> 1;
        const float u = normed(2 * i), v = normed(2 * i + 1);
        const float co = cs[2 * i], si = cs[2 * i + 1];
        return (d & 1) ? v * co + u * si : u * co - v * si;
    };
    for (int idx = tid; idx < nq * hd; idx += NT) {
        const int h = idx / hd, d = idx - h * hd;
        q_out[(size_t)t * nq * hd + idx] = hb_from_float<TQ>(turned(h * dim, d, inv_q));
    }
    for (int idx = tid; idx < nkv * hd; idx += NT) {
        const int g = idx / hd, d = idx - g * hd;
        const size_t base = ((size_t)page * nkv + g) * page_size * hd;
        k_cache[base + (size_t)in_page * hd + d] = hb_from_float<TC>(turned(QD + g * dim, d, inv_k));
        const float v = d < vdim ? filtered[QD + KD + g * vdim + d] : 0.f;
        v_cache[base + (size_t)d * page_size + in_page] = hb_from_float<TC>(v);
    }
}

extern "C" int hb_filter_norm_rotate_write(const float* proj, int ld, const float* taps, int K, float* filter_state,
                                           const float* q_norm_w, const float* k_norm_w, const double* rates,
                                           int rot_dims, const int* positions, const int* seq_of,
                                           const int* seq_starts, const int* slots, const int* page_table,
                                           int max_pages, int page_size, void* q_out, void* k_cache, void* v_cache,
                                           int dtype, int T, int nq, int nkv, int dim, int vdim, int hd, float eps,
                                           int longest, const float* bias, int head_norm, hipStream_t stream) {
    HB_REQUIRE(T > 0 && nq > 0 && nkv > 0 && dim > 0 && vdim > 0, "filtered attention: empty input");
    HB_REQUIRE(hd >= dim && hd >= vdim, "filtered attention: heads kept at %d cannot hold %d and %d", hd, dim, vdim);
    const long long C = (long long)(nq + nkv) * dim + (long long)nkv * vdim;
    HB_REQUIRE(ld >= C, "filtered attention: rows of %d do not hold %lld channels", ld, C);
    HB_REQUIRE(taps == nullptr || (K >= 1 && K <= 16), "filtered attention: %d taps, the kernel takes 1 to 16", K);
    HB_REQUIRE(taps == nullptr || K == 1 || filter_state != nullptr, "filtered attention: a filter needs its state");
    HB_REQUIRE(rates == nullptr || (rot_dims > 0 && rot_dims % 2 == 0 && rot_dims <= dim),
               "filtered attention: %d rotated entries of heads of %d", rot_dims, dim);
    HB_REQUIRE(!head_norm || (q_norm_w != nullptr && k_norm_w != nullptr), "filtered attention: a norm a head needs its weights");
    const size_t lds = ((size_t)C + (rates ? rot_dims : 0) + (head_norm ? nq + nkv : 0)) * sizeof(float);
    HB_REQUIRE(lds <= 60 * 1024, "filtered attention: %lld channels a token do not fit the kernel's LDS", C);
    if (taps == nullptr) K = 0;
    // longest: the most tokens that a sequence of the step brings; at one the kernel moves the filter's state on
    // itself, otherwise hb_filter_state does so afterwards
    const int moves_state = longest == 1 && K > 1;
#define HB_FNRW_NT(TQ, TC, TK, NT)                                                                                       \
    filter_norm_rotate_write_kernel<TQ, TC, TK, NT><<<T, NT, lds, stream>>>(                                              \
        proj, ld, taps, K, filter_state, q_norm_w, k_norm_w, rates, rot_dims, positions, seq_of, seq_starts, slots,       \
        page_table, max_pages, page_size, (TQ*)q_out, (TC*)k_cache, (TC*)v_cache, nq, nkv, dim, vdim, hd, eps,   \
        moves_state, bias, head_norm)
#define HB_FNRW(TQ, TC, TK)                                                                                              \
    do {                                                                                                                 \
        if (T <= 64) HB_FNRW_NT(TQ, TC, TK, 1024);                                                                       \
        else HB_FNRW_NT(TQ, TC, TK, 256);                                                                                \
    } while (0)
#define HB_FNRW_TAPS(TQ, TC)                                                                                             \
    do {                                                                                                                 \
        if (K == 4) HB_FNRW(TQ, TC, 4);                                                                                  \
        else if (K == 3) HB_FNRW(TQ, TC, 3);                                                                             \
        else if (K == 2) HB_FNRW(TQ, TC, 2);                                                                             \
        else HB_FNRW(TQ, TC, 0);                                                                                         \
    } while (0)
    if (dtype == HB_F32)
        HB_FNRW_TAPS(float, float);
    else if (dtype == HB_BF16)
        HB_FNRW_TAPS(bf16, bf16);
    else
        HB_REQUIRE(false, "filtered attention: unknown dtype %d", dtype);
#undef HB_FNRW_TAPS
#undef HB_FNRW
#undef HB_FNRW_NT
    HB_CHECK_LAUNCH("filter_norm_rotate_write");
    return 0;
}

// ------------------------------------------- a bias a column
// x[t, c] += bias[c]: the bias of a projection whose product adds to these rows.
__global__ void add_bias_kernel(float* __restrict__ x, const float* __restrict__ bias, int H, size_t total) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx < total) x[idx] += bias[idx % H];
}

extern "C" int hb_add_bias(float* x, const float* bias, int T, int H, hipStream_t stream) {
    HB_REQUIRE(T > 0 && H > 0, "bias: empty input");
    const size_t total = (size_t)T * H;
    add_bias_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(x, bias, H, total);
    HB_CHECK_LAUNCH("add_bias");
    return 0;
}

// ------------------------------------------- a gate on the heads' outputs
// out[t, h x vdim + d] = attn[t, h x hd + d] * sigmoid(gate[t, g_off + h x vdim + d]) for d < vdim: the heads'
// outputs, kept at size hd, leave at their own size, each entry times a gate of its own (gate_rows null: none).
template <class TIn, class TOut>
__global__ void gate_heads_kernel(const TIn* __restrict__ attn, const float* __restrict__ gate_rows, int ld, int g_off,
                                  TOut* __restrict__ out, int nq, int hd, int vdim, size_t total) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int W = nq * vdim;
    const size_t t = idx / W;
    const int c = (int)(idx - t * W);
    const int h = c / vdim, d = c - h * vdim;
    float v = hb_to_float(attn[(t * nq + h) * hd + d]);
    if (gate_rows) v *= 1.0f / (1.0f + expf(-gate_rows[t * ld + g_off + c]));
    out[idx] = hb_from_float<TOut>(v);
}

extern "C" int hb_gate_heads(const void* attn, int dtype, const float* gate_rows, int ld, int g_off, void* out, int T,
                             int nq, int hd, int vdim, hipStream_t stream) {
    HB_REQUIRE(T > 0 && nq > 0 && vdim > 0 && hd >= vdim, "gate: empty input or heads of %d kept at %d", vdim, hd);
    HB_REQUIRE(gate_rows == nullptr || (g_off >= 0 && g_off + nq * vdim <= ld), "gate: its columns lie outside the rows");
    const size_t total = (size_t)T * nq * vdim;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (dtype == HB_F32)
        gate_heads_kernel<float, float><<<blocks, 256, 0, stream>>>((const float*)attn, gate_rows, ld, g_off, (float*)out, nq, hd, vdim, total);
    else if (dtype == HB_BF16)
        gate_heads_kernel<bf16, bf16><<<blocks, 256, 0, stream>>>((const bf16*)attn, gate_rows, ld, g_off, (bf16*)out, nq, hd, vdim, total);
    else
        HB_REQUIRE(false, "gate: unknown dtype %d", dtype);
    HB_CHECK_LAUNCH("gate_heads");
    return 0;
}

// ------------------------------------------- a token's own input to the residual stream, layer by layer
// With e = table[token, col0 .. col0 + D) (a token's row of a table, this layer's part of it):
//     g = gelu_tanh(W_gate x) * e;   y = W_proj g;   x <- x + y / sqrt(mean(y^2) + eps) * w
// x f32 [T, H] in place; W_gate [D, H], the table, and W_proj transposed [D, H] in one storage type; all arithmetic
// float32. Three kernels, each of which fills the chip for a few tokens as for thousands:
//   gate: a workgroup takes SIDE_TOKENS tokens and 4 x RW rows of W_gate (RW = 4; eight rows a wave were no faster); a wave takes RW of them, its lanes
//     share a row's columns (whole lines of the matrix), every x is read once for the wave's RW rows; the sums
//     over the lanes run in a fixed order; g f32 [T, D]; a step of few tokens gives a row to a whole workgroup;
//   proj: a workgroup takes SIDE_TOKENS tokens (their g in LDS) and 64 columns of y; a lane takes a column,
//     its weights W_proj^T [j, c] lie side by side for neighbouring lanes, the four waves a quarter of the
//     gates each; y f32 [T, H];
//   add: a workgroup a token: the row's mean of squares in a fixed order, then x += y / rms * w.
#define SIDE_TOKENS 8
template <class TW, int RW>
__global__ void __launch_bounds__(256)
token_gate_kernel(const float* __restrict__ x, const int* __restrict__ tokens, const TW* __restrict__ table,
                  int table_ld, int col0, const TW* __restrict__ w_gate, float* __restrict__ g, bf16* __restrict__ g16,
                  int T, int H, int D) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t0 = blockIdx.y * SIDE_TOKENS;
    const int j0 = (blockIdx.x * 4 + wave) * RW;
    if (j0 >= D) return;
    float acc[RW][SIDE_TOKENS];
#pragma unroll
    for (int r = 0; r < RW; ++r)
#pragma unroll
        for (int k = 0; k < SIDE_TOKENS; ++k) acc[r][k] = 0.f;
    for (int c = lane; c < H; c += 64) {
        float w[RW], xv[SIDE_TOKENS];
#pragma unroll
        // (rows past the end read the last row again: a load under a condition would wait for the one before it,
        //  and what is summed for such a row is never stored)
        for (int r = 0; r < RW; ++r) w[r] = hb_to_float(w_gate[(size_t)(j0 + r < D ? j0 + r : D - 1) * H + c]);
#pragma unroll
        for (int k = 0; k < SIDE_TOKENS; ++k) xv[k] = x[(size_t)(t0 + k < T ? t0 + k : T - 1) * H + c];
#pragma unroll
        for (int r = 0; r < RW; ++r)
#pragma unroll
            for (int k = 0; k < SIDE_TOKENS; ++k) acc[r][k] = fmaf(w[r], xv[k], acc[r][k]);
    }
#pragma unroll
    for (int r = 0; r < RW; ++r)
#pragma unroll
        for (int k = 0; k < SIDE_TOKENS; ++k) {
            const float z = hb_wave_sum(acc[r][k]);
            if (lane == 0 && j0 + r < D && t0 + k < T) {
                const float gelu = 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
                const float out = gelu * hb_to_float(table[(size_t)tokens[t0 + k] * table_ld + col0 + j0 + r]);
                if (g16) g16[(size_t)(t0 + k) * D + j0 + r] = hb_from_float<bf16>(out);       // (for a product on the matrix cores)
                else g[(size_t)(t0 + k) * D + j0 + r] = out;
            }
        }
}

// (few tokens: all four waves of a workgroup share one row of W_gate, a quarter of its columns each)
template <class TW>
__global__ void __launch_bounds__(256)
token_gate_few_kernel(const float* __restrict__ x, const int* __restrict__ tokens, const TW* __restrict__ table,
                      int table_ld, int col0, const TW* __restrict__ w_gate, float* __restrict__ g, int T, int H, int D) {
    __shared__ float part[4][SIDE_TOKENS];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t0 = blockIdx.y * SIDE_TOKENS, j = blockIdx.x;
    float acc[SIDE_TOKENS];
#pragma unroll
    for (int k = 0; k < SIDE_TOKENS; ++k) acc[k] = 0.f;
#pragma unroll 4
    for (int c = threadIdx.x; c < H; c += 256) {
        const float w = hb_to_float(w_gate[(size_t)j * H + c]);
#pragma unroll
        for (int k = 0; k < SIDE_TOKENS; ++k) acc[k] = fmaf(w, x[(size_t)(t0 + k < T ? t0 + k : T - 1) * H + c], acc[k]);
    }
#pragma unroll
    for (int k = 0; k < SIDE_TOKENS; ++k) {
        const float z = hb_wave_sum(acc[k]);
        if (lane == 0) part[wave][k] = z;
    }
    __syncthreads();
    const int k = threadIdx.x;
    if (k < SIDE_TOKENS && t0 + k < T) {
        const float z = ((part[0][k] + part[1][k]) + part[2][k]) + part[3][k];
        const float gelu = 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
        g[(size_t)(t0 + k) * D + j] = gelu * hb_to_float(table[(size_t)tokens[t0 + k] * table_ld + col0 + j]);
    }
}

// (64 columns of y a workgroup; wave q takes the q-th quarter of the D gates, and the four partial sums of a
// column are added in their order)
template <class TW>
__global__ void __launch_bounds__(256)
token_proj_kernel(const float* __restrict__ g, const TW* __restrict__ w_proj_t, float* __restrict__ y, int T, int H,
                  int D) {
    extern __shared__ float side_g[];              // [SIDE_TOKENS][D], then the partial sums [3][SIDE_TOKENS][64]
    float* const partial = side_g + SIDE_TOKENS * D;
    const int t0 = blockIdx.y * SIDE_TOKENS;
    const int lane = threadIdx.x & 63, q = threadIdx.x >> 6;
    const int c = blockIdx.x * 64 + lane;
    for (int i = threadIdx.x; i < SIDE_TOKENS * D; i += 256) {
        const int k = i / D;
        side_g[i] = t0 + k < T ? g[(size_t)(t0 + k) * D + (i - k * D)] : 0.f;
    }
    __syncthreads();
    const int per = (D + 3) / 4;
    const int j0 = q * per, j1 = j0 + per < D ? j0 + per : D;
    float acc[SIDE_TOKENS];
#pragma unroll
    for (int k = 0; k < SIDE_TOKENS; ++k) acc[k] = 0.f;
    if (c < H) {
        // sixteen weights asked for at once (one after the other, each would wait for memory), then their products
        for (int j = j0; j < j1; j += 16) {
            float w[16];
#pragma unroll
            // (no load stands under a condition, which would make it wait for the one before: past the end the last
            //  weight is read again and counts as zero)
            for (int o = 0; o < 16; ++o) w[o] = hb_to_float(w_proj_t[(size_t)(j + o < j1 ? j + o : j1 - 1) * H + c]);
#pragma unroll
            for (int o = 0; o < 16; ++o) {
                const int at = j + o < j1 ? j + o : j1 - 1;
                const float wo = j + o < j1 ? w[o] : 0.f;
#pragma unroll
                for (int k = 0; k < SIDE_TOKENS; ++k) acc[k] = fmaf(wo, side_g[k * D + at], acc[k]);
            }
        }
    }
    if (q > 0) {
#pragma unroll
        for (int k = 0; k < SIDE_TOKENS; ++k) partial[((q - 1) * SIDE_TOKENS + k) * 64 + lane] = acc[k];
    }
    __syncthreads();
    if (q > 0 || c >= H) return;
#pragma unroll
    for (int k = 0; k < SIDE_TOKENS; ++k) {
        float sum = acc[k];
#pragma unroll
        for (int o = 0; o < 3; ++o) sum += partial[(o * SIDE_TOKENS + k) * 64 + lane];
        if (t0 + k < T) y[(size_t)(t0 + k) * H + c] = sum;
    }
}

__global__ void __launch_bounds__(256)
add_normed_kernel(float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ w, int H, float eps) {
    __shared__ float red[16];
    const size_t row = (size_t)blockIdx.x * H;
    float ss = 0.f;
    for (int c = threadIdx.x; c < H; c += 256) ss = fmaf(y[row + c], y[row + c], ss);
    ss = hb_block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
    for (int c = threadIdx.x; c < H; c += 256) x[row + c] += y[row + c] * inv * w[c];
}

// g f32 [T, D] and y f32 [T, H] are the caller's scratch. stage 1: all three kernels. stage 0: the gate alone,
// which leaves g as bfloat16 in g16 [T, D] if that is given (many tokens only): the caller's own product makes y
// from it; stage 2: the norm and the sum alone, from the caller's y.
extern "C" int hb_token_side(float* x, const int* tokens, const void* table, int table_ld, int col0, const void* w_gate,
                             const void* w_proj_t, int dtype, const float* norm_w, float* g, void* g16v, float* y, int T,
                             int H, int D, float eps, int stage, hipStream_t stream) {
    bf16* const g16 = (bf16*)g16v;
    if (stage == 2) {
        HB_REQUIRE(T > 0 && H > 0, "token input: empty input");
        add_normed_kernel<<<T, 256, 0, stream>>>(x, y, norm_w, H, eps);
        HB_CHECK_LAUNCH("token_add_normed");
        return 0;
    }
    HB_REQUIRE(T > 0 && H > 0 && D > 0, "token input: empty input");
    HB_REQUIRE(col0 >= 0 && col0 + D <= table_ld, "token input: the layer's columns lie outside the table's rows");
    const size_t lds = ((size_t)SIDE_TOKENS * D + 3 * SIDE_TOKENS * 64) * sizeof(float);
    HB_REQUIRE(lds <= 60 * 1024, "token input: %d gates a token do not fit the kernel's LDS", D);
    const int tiles = (T + SIDE_TOKENS - 1) / SIDE_TOKENS;
    HB_REQUIRE(tiles <= 65535, "token input: too many tokens for the grid");
    const bool many = T > 64;          // (few tokens: a row a workgroup, so that the gate's rows are spread over more waves)
    HB_REQUIRE(g16 == nullptr || (many && stage == 0), "token input: bfloat16 gates are for many tokens and a product of the caller's");
    HB_REQUIRE(D <= 65535, "token input: too many gates for the grid");
#define HB_SIDE(TW)                                                                                                   \
    do {                                                                                                              \
        if (many)                                                                                                     \
            token_gate_kernel<TW, 4><<<dim3((D + 15) / 16, tiles), 256, 0, stream>>>(                                  \
                x, tokens, (const TW*)table, table_ld, col0, (const TW*)w_gate, g, g16, T, H, D);                     \
        else                                                                                                          \
            token_gate_few_kernel<TW><<<dim3(D, tiles), 256, 0, stream>>>(                                             \
                x, tokens, (const TW*)table, table_ld, col0, (const TW*)w_gate, g, T, H, D);                          \
        HB_CHECK_LAUNCH("token_gate");                                                                                \
        if (stage != 1) break;                                                                                        \
        token_proj_kernel<TW><<<dim3((H + 63) / 64, tiles), 256, lds, stream>>>(g, (const TW*)w_proj_t, y, T, H, D);   \
        HB_CHECK_LAUNCH("token_proj");                                                                                \
    } while (0)
    if (dtype == HB_F32) HB_SIDE(float);
    else if (dtype == HB_BF16) HB_SIDE(bf16);
    else HB_REQUIRE(false, "token input: unknown dtype %d", dtype);
#undef HB_SIDE
    if (stage != 1) return 0;
    add_normed_kernel<<<T, 256, 0, stream>>>(x, y, norm_w, H, eps);
    HB_CHECK_LAUNCH("token_add_normed");
    return 0;
}
