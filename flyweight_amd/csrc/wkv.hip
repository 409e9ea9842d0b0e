// A linear recurrence over a matrix state per head with a decay per key channel that the token itself
// forms and a bonus for the current token ("wkv"), and the mixing of a token's input with the input of the
// token before it that stands in front of it. All arithmetic float32, whatever the run's dtype.
//
//   o_t = (S + diag(u) k_t v_t^T)^T r_t = S^T r_t + (sum_c r_t[c] u[c] k_t[c]) v_t
//   S  <- diag(w_t) S + k_t v_t^T,            w_t = exp(-exp(a_t + w0))
//
// S [key channel][value channel] per head and request, zero at a request's start.
#include "fw_common.h"
#include "fw_kernels.h"

// ---- token shift --------------------------------------------------------------------------------
// A workgroup per row. h = x * rsqrt(mean(x^2) + eps) * (w or 1 + w) (norm_weight null: h = x). The row
// before comes from the same step (normed again here: a row is read twice, nothing is kept between
// workgroups) or, for a segment's first row, from the request's slot. out[s][row] = h + (before - h) *
// mu[s]. The workgroup of a segment's FIRST row also moves the slot on to the h of the segment's LAST
// row: it alone reads and writes the slot, each thread its own channels, the read first.
template <typename T>
__global__ __launch_bounds__(256) void token_shift_mix_kernel(
    const float* __restrict__ x, const float* __restrict__ norm_weight, float eps, int one_centered,
    const float* __restrict__ mu, int mixes, float* __restrict__ last, const int32_t* __restrict__ row_seg,
    const int32_t* __restrict__ seg_row0, const int32_t* __restrict__ seg_slot, T* __restrict__ out, int rows, int hidden) {
    __shared__ float scratch[16];
    const int row = blockIdx.x;
    const int seg = row_seg[row];
    const int first_row = seg_row0[seg], last_row = seg_row0[seg + 1] - 1;
    const bool is_first = row == first_row;
    float* slot = last + (size_t)seg_slot[seg] * hidden;
    auto inverse_rms = [&](const float* source) {
        if (!norm_weight) return 1.0f;
        float sum = 0.0f;
        for (int i = threadIdx.x; i < hidden; i += 256) sum += source[i] * source[i];
        sum = block_sum(sum, scratch);
        return rsqrtf(sum / (float)hidden + eps);
    };
    const float* mine = x + (size_t)row * hidden;
    const float* other = x + (size_t)(is_first ? last_row : row - 1) * hidden;     // a first row: the row that the slot will hold
    const float inv = inverse_rms(mine);
    const float inv_other = (is_first && last_row == row) ? inv : inverse_rms(other);
    for (int i = threadIdx.x; i < hidden; i += 256) {
        const float w = norm_weight ? (one_centered ? 1.0f + norm_weight[i] : norm_weight[i]) : 1.0f;
        const float h = mine[i] * inv * w;
        const float h_other = other[i] * inv_other * w;
        float before = h_other;
        if (is_first) {
            before = slot[i];
            slot[i] = h_other;
        }
        for (int s = 0; s < mixes; ++s)
            store_from_float(out, ((size_t)s * rows + row) * hidden + i, fmaf(before - h, mu[(size_t)s * hidden + i], h));
    }
}

extern "C" int fw_token_shift_mix(const float* x, const float* norm_weight, float eps, int one_centered, const float* mu, int mixes,
                                  float* last, int slots, const int32_t* row_seg, const int32_t* seg_row0, const int32_t* seg_slot,
                                  void* out, int out_dtype, int rows, int segments, int hidden, void* stream) {
    FW_REQUIRE(rows >= 0 && segments >= 0 && hidden > 0 && mixes > 0 && slots > 0, "token_shift_mix: bad sizes rows=%d segments=%d hidden=%d mixes=%d",
               rows, segments, hidden, mixes);
    FW_REQUIRE(rows <= 1 << 20, "token_shift_mix: too many rows (%d)", rows);
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (out_dtype == FW_F32)
        token_shift_mix_kernel<float><<<rows, 256, 0, s>>>(x, norm_weight, eps, one_centered, mu, mixes, last, row_seg, seg_row0, seg_slot,
                                                           (float*)out, rows, hidden);
    else if (out_dtype == FW_BF16)
        token_shift_mix_kernel<bf16_t><<<rows, 256, 0, s>>>(x, norm_weight, eps, one_centered, mu, mixes, last, row_seg, seg_row0, seg_slot,
                                                            (bf16_t*)out, rows, hidden);
    else
        FW_REQUIRE(false, "token_shift_mix: unknown dtype %d", out_dtype);
    FW_LAUNCH_CHECK("token_shift_mix");
    return 0;
}

// out = tanh(x), float32 in, any dtype out
template <typename T>
__global__ void tanh_rows_kernel(const float* __restrict__ x, T* __restrict__ out, long long count) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (long long)gridDim.x * blockDim.x)
        store_from_float(out, (size_t)i, tanhf(x[i]));
}

extern "C" int fw_tanh_rows(const float* x, void* out, int out_dtype, long long count, void* stream) {
    FW_REQUIRE(count >= 0, "tanh_rows: negative count");
    if (count == 0) return 0;
    const int blocks = (int)((count + 255) / 256 > 4096 ? 4096 : (count + 255) / 256);
    if (out_dtype == FW_F32) tanh_rows_kernel<float><<<blocks, 256, 0, (hipStream_t)stream>>>(x, (float*)out, count);
    else if (out_dtype == FW_BF16) tanh_rows_kernel<bf16_t><<<blocks, 256, 0, (hipStream_t)stream>>>(x, (bf16_t*)out, count);
    else FW_REQUIRE(false, "tanh_rows: unknown dtype %d", out_dtype);
    FW_LAUNCH_CHECK("tanh_rows");
    return 0;
}

// ---- the recurrence ------------------------------------------------------------------------------
// A wave per (segment, head, 16 value channels). Lane = 16 p + c: value channel c of the tile, key
// channels p, p + 4, p + 8, ... (KPT of them: a quarter of the head's, interleaved so that the four lanes
// of a column read neighbouring words of LDS). A column's sum over key channels is each lane's own sum and
// then the four lanes' (two row swaps). Tokens come in chunks of WKV_CHUNK: the wave stages a chunk's r, k
// and decays in LDS (the decay's two exponentials are taken here, once per chunk and key channel), forms
// each token's bonus sum r . (u k), and then walks the chunk token by token. The state is read at the
// segment's start and written at its end. Columns of S never meet, so the result does not depend on how
// the work is cut; tokens are walked in order whatever the segments, so it does not depend on the cut of
// the sequence either.
#define WKV_CHUNK 16
template <int KPT>
__global__ __launch_bounds__(64) void wkv_recurrence_kernel(
    const float* __restrict__ r, const float* __restrict__ k, const float* __restrict__ v, int rkv_stride,
    const float* __restrict__ a, int a_stride, const float* __restrict__ w0, const float* __restrict__ u, float* __restrict__ state,
    float* __restrict__ out, const int32_t* __restrict__ seg_row0, const int32_t* __restrict__ seg_slot, int heads, int dim) {
    extern __shared__ float lds[];
    const int padded = KPT * 4;                     // key channels as the lanes hold them
    float* rs = lds;                                // [WKV_CHUNK][padded]
    float* ks = rs + WKV_CHUNK * padded;
    float* ws = ks + WKV_CHUNK * padded;
    float* bonus = ws + WKV_CHUNK * padded;         // [WKV_CHUNK]
    const int seg = blockIdx.x, head = blockIdx.y, tile = blockIdx.z;
    const int lane = threadIdx.x, c = lane & 15, p = lane >> 4;
    const int column = tile * 16 + c;
    const bool column_there = column < dim;
    const int row0 = seg_row0[seg], row_end = seg_row0[seg + 1];
    float* S = state + ((size_t)seg_slot[seg] * heads + head) * dim * dim;
    float s[KPT];
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
        const int key = 4 * i + p;
        s[i] = (key < dim && column_there) ? S[(size_t)key * dim + column] : 0.0f;
    }
    const size_t head_at = (size_t)head * dim;
    for (int chunk0 = row0; chunk0 < row_end; chunk0 += WKV_CHUNK) {
        const int count = row_end - chunk0 < WKV_CHUNK ? row_end - chunk0 : WKV_CHUNK;
        for (int item = lane; item < count * padded; item += 64) {
            const int t = item / padded, key = item % padded;
            const size_t row = chunk0 + t;
            float rv = 0.0f, kv = 0.0f, wv = 0.0f;
            if (key < dim) {
                rv = r[row * rkv_stride + head_at + key];
                kv = k[row * rkv_stride + head_at + key];
                wv = expf(-expf(a[row * a_stride + head_at + key] + w0[head_at + key]));
            }
            rs[item] = rv;
            ks[item] = kv;
            ws[item] = wv;
        }
        fw_lds_barrier();
        for (int t = 0; t < count; ++t) {
            float part = 0.0f;
            for (int key = lane; key < dim; key += 64) part = fmaf(rs[t * padded + key] * u[head_at + key], ks[t * padded + key], part);
            part = wave_sum(part);
            if (lane == 0) bonus[t] = part;
        }
        fw_lds_barrier();
        for (int t = 0; t < count; ++t) {
            const size_t row = chunk0 + t;
            const float value = column_there ? v[row * rkv_stride + head_at + column] : 0.0f;
            const float* rt = rs + t * padded;
            const float* kt = ks + t * padded;
            const float* wt = ws + t * padded;
            float sum = 0.0f;
#pragma unroll
            for (int i = 0; i < KPT; ++i) {
                const int key = 4 * i + p;
                sum = fmaf(rt[key], s[i], sum);
                s[i] = fmaf(wt[key], s[i], kt[key] * value);
            }
            sum = fw_quad_sum(sum);
            if (p == 0 && column_there) out[row * (size_t)heads * dim + head_at + column] = fmaf(bonus[t], value, sum);
        }
        fw_lds_barrier();       // the next chunk overwrites what this walk has read
    }
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
        const int key = 4 * i + p;
        if (key < dim && column_there) S[(size_t)key * dim + column] = s[i];
    }
}

extern "C" int fw_wkv_recurrence(const float* r, const float* k, const float* v, int rkv_stride, const float* a, int a_stride,
                                 const float* w0, const float* u, float* state, int slots, float* out, const int32_t* seg_row0,
                                 const int32_t* seg_slot, int rows, int segments, int heads, int dim, void* stream) {
    FW_REQUIRE(rows >= 0 && segments >= 0 && heads > 0 && heads <= 65535 && slots > 0, "wkv_recurrence: bad sizes rows=%d segments=%d heads=%d", rows, segments, heads);
    FW_REQUIRE(dim >= 1 && dim <= 256, "wkv_recurrence: a head of %d channels (1..256)", dim);
    FW_REQUIRE(rkv_stride >= heads * dim && a_stride >= heads * dim, "wkv_recurrence: rows of %d / %d values do not hold %d heads of %d", rkv_stride, a_stride, heads, dim);
    if (rows == 0 || segments == 0) return 0;
    dim3 grid(segments, heads, (dim + 15) / 16);
    hipStream_t s = (hipStream_t)stream;
#define FW_WKV_LAUNCH(KPT)                                                                                                     \
    {                                                                                                                          \
        const int lds_bytes = (3 * WKV_CHUNK * KPT * 4 + WKV_CHUNK) * 4;                                                       \
        static int configured = 0;                                                                                             \
        if (lds_bytes > 48 * 1024 && lds_bytes > configured) {                                                                 \
            hipError_t status = hipFuncSetAttribute((const void*)wkv_recurrence_kernel<KPT>,                                   \
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);                    \
            FW_REQUIRE(status == hipSuccess, "wkv_recurrence: cannot reserve %d bytes of LDS", lds_bytes);                     \
            configured = lds_bytes;                                                                                            \
        }                                                                                                                      \
        wkv_recurrence_kernel<KPT><<<grid, 64, lds_bytes, s>>>(r, k, v, rkv_stride, a, a_stride, w0, u, state, out, seg_row0,  \
                                                               seg_slot, heads, dim);                                         \
    }
    if (dim <= 32) FW_WKV_LAUNCH(8)
    else if (dim <= 64) FW_WKV_LAUNCH(16)
    else if (dim <= 128) FW_WKV_LAUNCH(32)
    else FW_WKV_LAUNCH(64)
#undef FW_WKV_LAUNCH
    FW_LAUNCH_CHECK("wkv_recurrence");
    return 0;
}
