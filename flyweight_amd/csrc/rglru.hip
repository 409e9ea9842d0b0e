// A short causal convolution per channel over mixed segments, and the real-gated linear recurrence per
// channel ("RG-LRU") that reads it.
//
//   fw_causal_conv   y[t][c] = sum_j taps[c][j] * x[t - L + 1 + j][c] (+ bias[c]), the inputs before a segment's first
//                    row from the request's slot (zeros for a new request), which is then moved on
//   fw_rglru_scan    r = sigmoid(gr + br), i = sigmoid(gi + bi), a = exp(-rate r softplus(lam)),
//                    S <- a S + sqrt(1 - a^2) i u, out = S * gelu_tanh(y)
//
// Everything here is float32 whatever the run's dtype; the recurrence walks a segment's rows in order, so a
// position's result does not depend on how the sequence was cut into steps.
#include "fw_common.h"
#include "fw_kernels.h"

#define CONV_MAX_TAPS 16

// ---- the convolution -------------------------------------------------------------------------------------
// Outputs: a thread per (row, channel). The input t rows back is the step's own row where the segment reaches
// that far, else what the slot remembers: state [slots][channels][L - 1], oldest first. Channels echo_col0 ..
// echo_col0 + echo_cols - 1 are written a second time, from column echo_to on (a consumer that wants them twice).
__global__ __launch_bounds__(256) void causal_conv_rows_kernel(
    const float* __restrict__ in, int in_stride, const float* __restrict__ taps, const float* __restrict__ bias,
    const float* __restrict__ state, const int32_t* __restrict__ row_seg, const int32_t* __restrict__ seg_row0,
    const int32_t* __restrict__ seg_slot, float* __restrict__ out, int out_stride, int echo_col0, int echo_cols, int echo_to,
    int rows, int channels, int L) {
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    const int row = blockIdx.x;
    if (c >= channels) return;
    const int seg = row_seg[row];
    const int first = seg_row0[seg];
    const float* remembered = state + ((size_t)seg_slot[seg] * channels + c) * (L - 1);
    float sum = bias ? bias[c] : 0.0f;
    for (int j = 0; j < L; ++j) {
        const int t = row - (L - 1) + j;
        const float x = t >= first ? in[(size_t)t * in_stride + c] : remembered[(L - 1) + (t - first)];
        sum = fmaf(taps[(size_t)c * L + j], x, sum);
    }
    out[(size_t)row * out_stride + c] = sum;
    if (c >= echo_col0 && c < echo_col0 + echo_cols) out[(size_t)row * out_stride + echo_to + (c - echo_col0)] = sum;
}

// The slots move on: a thread per (segment, channel) reads what it needs (the segment's last L - 1 inputs, of
// which the slot's own newest ones stand in for rows the segment does not have) and then writes.
__global__ __launch_bounds__(256) void causal_conv_state_kernel(
    const float* __restrict__ in, int in_stride, float* __restrict__ state, const int32_t* __restrict__ seg_row0,
    const int32_t* __restrict__ seg_slot, int channels, int L) {
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    const int seg = blockIdx.x;
    if (c >= channels) return;
    const int first = seg_row0[seg], end = seg_row0[seg + 1];
    float* remembered = state + ((size_t)seg_slot[seg] * channels + c) * (L - 1);
    float keep[CONV_MAX_TAPS - 1];
#pragma unroll
    for (int i = 0; i < CONV_MAX_TAPS - 1; ++i) {
        if (i >= L - 1) break;
        const int t = end - (L - 1) + i;
        keep[i] = t >= first ? in[(size_t)t * in_stride + c] : remembered[(L - 1) + (t - first)];
    }
#pragma unroll
    for (int i = 0; i < CONV_MAX_TAPS - 1; ++i) {
        if (i >= L - 1) break;
        remembered[i] = keep[i];
    }
}

// Every segment is one row (a decode step): output and the slot's move in one launch, a thread per (row, channel).
__global__ __launch_bounds__(256) void causal_conv_step_kernel(
    const float* __restrict__ in, int in_stride, const float* __restrict__ taps, const float* __restrict__ bias,
    float* __restrict__ state, const int32_t* __restrict__ seg_slot, float* __restrict__ out, int out_stride, int echo_col0,
    int echo_cols, int echo_to, int channels, int L) {
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    const int row = blockIdx.x;
    if (c >= channels) return;
    float* remembered = state + ((size_t)seg_slot[row] * channels + c) * (L - 1);
    const float x = in[(size_t)row * in_stride + c];
    float sum = bias ? bias[c] : 0.0f;
    float keep[CONV_MAX_TAPS - 1];
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS - 1; ++j) {
        if (j >= L - 1) break;
        keep[j] = remembered[j];
        sum = fmaf(taps[(size_t)c * L + j], keep[j], sum);
    }
    sum = fmaf(taps[(size_t)c * L + L - 1], x, sum);
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS - 1; ++j) {
        if (j >= L - 1) break;
        remembered[j] = j + 1 < L - 1 ? keep[j + 1] : x;
    }
    out[(size_t)row * out_stride + c] = sum;
    if (c >= echo_col0 && c < echo_col0 + echo_cols) out[(size_t)row * out_stride + echo_to + (c - echo_col0)] = sum;
}

extern "C" int fw_causal_conv(const float* in, int in_stride, const float* taps, const float* bias, float* state,
                              const int32_t* row_seg, const int32_t* seg_row0, const int32_t* seg_slot, float* out, int out_stride,
                              int echo_col0, int echo_cols, int echo_to, int rows, int segments, int channels, int taps_count,
                              int slots, int single_rows, void* stream) {
    FW_REQUIRE(rows >= 0 && segments >= 0 && channels > 0 && slots > 0, "causal_conv: bad sizes rows=%d segments=%d channels=%d slots=%d",
               rows, segments, channels, slots);
    FW_REQUIRE(taps_count >= 1 && taps_count <= CONV_MAX_TAPS, "causal_conv: %d taps (1..%d)", taps_count, CONV_MAX_TAPS);
    FW_REQUIRE(in_stride >= channels && out_stride >= channels, "causal_conv: rows %d / %d wide do not hold %d channels", in_stride,
               out_stride, channels);
    FW_REQUIRE(echo_cols >= 0 && (echo_cols == 0 || (echo_col0 >= 0 && echo_col0 + echo_cols <= channels && echo_to >= channels &&
                                                      echo_to + echo_cols <= out_stride)),
               "causal_conv: channels %d..%d cannot be written again from column %d of rows %d wide", echo_col0, echo_col0 + echo_cols,
               echo_to, out_stride);
    FW_REQUIRE(!single_rows || rows == segments, "causal_conv: %d rows are not %d segments of one row", rows, segments);
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const unsigned across = (unsigned)fw_ceil_div(channels, 256);
    if (single_rows) {
        causal_conv_step_kernel<<<dim3(rows, across), 256, 0, s>>>(in, in_stride, taps, bias, state, seg_slot, out, out_stride, echo_col0,
                                                                   echo_cols, echo_to, channels, taps_count);
        FW_LAUNCH_CHECK("causal_conv");
        return 0;
    }
    causal_conv_rows_kernel<<<dim3(rows, across), 256, 0, s>>>(in, in_stride, taps, bias, state, row_seg, seg_row0, seg_slot, out,
                                                               out_stride, echo_col0, echo_cols, echo_to, rows, channels, taps_count);
    FW_LAUNCH_CHECK("causal_conv");
    if (taps_count > 1) {
        causal_conv_state_kernel<<<dim3(segments, across), 256, 0, s>>>(in, in_stride, state, seg_row0, seg_slot, channels, taps_count);
        FW_LAUNCH_CHECK("causal_conv (state)");
    }
    return 0;
}

// ---- the recurrence ----------------------------------------------------------------------------------------
// A thread per (segment, channel); neighbouring lanes hold neighbouring channels, so every load of a row is one
// run of memory. Rows are taken SCAN_ROWS at a time: their inputs are asked for together and everything that does
// not depend on the state (the gates, the decay, the input's weight, the gelu of the other branch) is formed for all
// of them before the chain S <- a S + b walks them.
#define SCAN_ROWS 8

__device__ __forceinline__ float rglru_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float rglru_gelu_tanh(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// What a row adds to the recurrence, from its inputs: the decay a and the weighted input b of S <- a S + b.
// 1 - a^2 is formed as -expm1(2 log a): a channel that barely forgets has a near 1, where 1 - a * a would lose its digits.
__device__ __forceinline__ void rglru_step_terms(float u, float gr, float gi, float br, float bi, float decay, float& a, float& b) {
    const float r = rglru_sigmoid(gr + br), i = rglru_sigmoid(gi + bi);
    a = expf(decay * r);
    b = sqrtf(-expm1f(2.0f * decay * r)) * (i * u);
}

// Segments of more than SCAN_LONG rows are walked in chunks of SCAN_CHUNK rows side by side, in two launches. The first
// walks every chunk on its own (the segment's first chunk from the slot's state, the others from zero) and leaves per row
// the chunk's state so far (local) and the product of its decays so far (carry): S_t = carry_t * S_in + local_t with S_in
// the state at the chunk's start. The second finds S_in from the chunks before (their last rows' carry and local, a few
// dozen steps), finishes the rows and moves the slot on. Shorter segments keep the walk in order above, whose sums do not
// depend on how a sequence is cut; a long one's differ from it by rounding alone.
#define SCAN_LONG 256
#define SCAN_CHUNK 64

__global__ __launch_bounds__(64) void rglru_chunk_local_kernel(
    const float* __restrict__ u, int u_stride, const float* __restrict__ gates, int gates_stride, const float* __restrict__ r_bias,
    const float* __restrict__ i_bias, const float* __restrict__ lam, float rate, const float* __restrict__ state,
    const int32_t* __restrict__ seg_row0, const int32_t* __restrict__ seg_slot, float* __restrict__ local, float* __restrict__ carry,
    int channels, int block_width) {
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    const int seg = blockIdx.x, chunk = blockIdx.z;
    const int first = seg_row0[seg], end = seg_row0[seg + 1];
    if (end - first <= SCAN_LONG || first + chunk * SCAN_CHUNK >= end || c >= channels) return;
    const int row_begin = first + chunk * SCAN_CHUNK;
    const int row_end = row_begin + SCAN_CHUNK < end ? row_begin + SCAN_CHUNK : end;
    const int block = c / block_width, within = c % block_width;
    const int r_col = block * 2 * block_width + within, i_col = r_col + block_width;
    const float br = r_bias[c], bi = i_bias[c];
    const float l = lam[c];
    const float decay = -rate * (l > 20.0f ? l : log1pf(expf(l)));
    float S = chunk == 0 ? state[(size_t)seg_slot[seg] * channels + c] : 0.0f;
    float product = 1.0f;
    for (int row0 = row_begin; row0 < row_end; row0 += SCAN_ROWS) {
        float uu[SCAN_ROWS], gr[SCAN_ROWS], gi[SCAN_ROWS];
#pragma unroll
        for (int k = 0; k < SCAN_ROWS; ++k) {
            const int row = row0 + k < row_end ? row0 + k : row_end - 1;
            uu[k] = u[(size_t)row * u_stride + c];
            gr[k] = gates[(size_t)row * gates_stride + r_col];
            gi[k] = gates[(size_t)row * gates_stride + i_col];
        }
        float a[SCAN_ROWS], b[SCAN_ROWS];
#pragma unroll
        for (int k = 0; k < SCAN_ROWS; ++k) rglru_step_terms(uu[k], gr[k], gi[k], br, bi, decay, a[k], b[k]);
#pragma unroll
        for (int k = 0; k < SCAN_ROWS; ++k) {
            if (row0 + k >= row_end) break;
            S = fmaf(a[k], S, b[k]);
            product *= a[k];
            local[(size_t)(row0 + k) * channels + c] = S;
            carry[(size_t)(row0 + k) * channels + c] = product;
        }
    }
}

template <typename TO>
__global__ __launch_bounds__(64) void rglru_chunk_finish_kernel(
    const float* __restrict__ y, int y_stride, const float* __restrict__ local, const float* __restrict__ carry, float* __restrict__ state,
    const int32_t* __restrict__ seg_row0, const int32_t* __restrict__ seg_slot, TO* __restrict__ out, int channels) {
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    const int seg = blockIdx.x, chunk = blockIdx.z;
    const int first = seg_row0[seg], end = seg_row0[seg + 1];
    if (end - first <= SCAN_LONG || first + chunk * SCAN_CHUNK >= end || c >= channels) return;
    const int row_begin = first + chunk * SCAN_CHUNK;
    const int row_end = row_begin + SCAN_CHUNK < end ? row_begin + SCAN_CHUNK : end;
    // the state at this chunk's start: through the chunks before it, in order (the first one holds the slot's state already)
    float S_in = 0.0f;
    for (int k = 0; k < chunk; ++k) {
        const size_t last = (size_t)(first + (k + 1) * SCAN_CHUNK - 1) * channels + c;
        S_in = k == 0 ? local[last] : fmaf(carry[last], S_in, local[last]);
    }
    float S = S_in;
    for (int row0 = row_begin; row0 < row_end; row0 += SCAN_ROWS) {
        float ll[SCAN_ROWS], cc[SCAN_ROWS], yy[SCAN_ROWS];
#pragma unroll
        for (int k = 0; k < SCAN_ROWS; ++k) {
            const int row = row0 + k < row_end ? row0 + k : row_end - 1;
            ll[k] = local[(size_t)row * channels + c];
            cc[k] = carry[(size_t)row * channels + c];
            yy[k] = y[(size_t)row * y_stride + c];
        }
#pragma unroll
        for (int k = 0; k < SCAN_ROWS; ++k) {
            if (row0 + k >= row_end) break;
            S = chunk == 0 ? ll[k] : fmaf(cc[k], S_in, ll[k]);
            store_from_float(out, (size_t)(row0 + k) * channels + c, S * rglru_gelu_tanh(yy[k]));
        }
    }
    if (row_end == end) state[(size_t)seg_slot[seg] * channels + c] = S;
}

template <typename TO>
__global__ __launch_bounds__(64) void rglru_scan_kernel(
    const float* __restrict__ u, int u_stride, const float* __restrict__ gates, int gates_stride, const float* __restrict__ y,
    int y_stride, const float* __restrict__ r_bias, const float* __restrict__ i_bias, const float* __restrict__ lam, float rate,
    float* __restrict__ state, const int32_t* __restrict__ seg_row0, const int32_t* __restrict__ seg_slot, TO* __restrict__ out,
    int channels, int block_width, int long_apart) {
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    const int seg = blockIdx.x;
    if (c >= channels) return;
    const int first = seg_row0[seg], end = seg_row0[seg + 1];
    if (long_apart && end - first > SCAN_LONG) return;      // the chunked kernels take it
    float* slot = state + (size_t)seg_slot[seg] * channels + c;
    // the gates of channel c lie block by block: [r of the block | i of the block]
    const int block = c / block_width, within = c % block_width;
    const int r_col = block * 2 * block_width + within, i_col = r_col + block_width;
    const float br = r_bias[c], bi = i_bias[c];
    const float l = lam[c];
    const float decay = -rate * (l > 20.0f ? l : log1pf(expf(l)));       // -rate * softplus(lam)
    float S = *slot;
    for (int row0 = first; row0 < end; row0 += SCAN_ROWS) {
        float uu[SCAN_ROWS], gr[SCAN_ROWS], gi[SCAN_ROWS], yy[SCAN_ROWS];
#pragma unroll
        for (int k = 0; k < SCAN_ROWS; ++k) {
            const int row = row0 + k < end ? row0 + k : end - 1;
            uu[k] = u[(size_t)row * u_stride + c];
            gr[k] = gates[(size_t)row * gates_stride + r_col];
            gi[k] = gates[(size_t)row * gates_stride + i_col];
            yy[k] = y[(size_t)row * y_stride + c];
        }
        float a[SCAN_ROWS], b[SCAN_ROWS];
#pragma unroll
        for (int k = 0; k < SCAN_ROWS; ++k) {
            rglru_step_terms(uu[k], gr[k], gi[k], br, bi, decay, a[k], b[k]);
            yy[k] = rglru_gelu_tanh(yy[k]);
        }
#pragma unroll
        for (int k = 0; k < SCAN_ROWS; ++k) {
            if (row0 + k >= end) break;
            S = fmaf(a[k], S, b[k]);
            store_from_float(out, (size_t)(row0 + k) * channels + c, S * yy[k]);
        }
    }
    *slot = S;
}

extern "C" int fw_rglru_scan(const float* u, int u_stride, const float* gates, int gates_stride, const float* y, int y_stride,
                             const float* r_bias, const float* i_bias, const float* lam, float rate, float* state,
                             const int32_t* seg_row0, const int32_t* seg_slot, void* out, int out_dtype, int rows, int segments,
                             int channels, int block_width, int slots, float* workspace, void* stream) {
    FW_REQUIRE(rows >= 0 && segments >= 0 && channels > 0 && slots > 0,
               "rglru_scan: bad sizes rows=%d segments=%d channels=%d slots=%d", rows, segments, channels, slots);
    FW_REQUIRE(block_width > 0 && channels % block_width == 0, "rglru_scan: %d channels are not blocks of %d", channels, block_width);
    FW_REQUIRE(u_stride >= channels && y_stride >= channels && gates_stride >= 2 * channels,
               "rglru_scan: rows %d / %d / %d wide do not hold %d channels (and twice as many gates)", u_stride, y_stride, gates_stride, channels);
    FW_REQUIRE(rate > 0.0f, "rglru_scan: the decay's rate must be positive");
    if (rows == 0 || segments == 0) return 0;
    FW_REQUIRE(out_dtype == FW_F32 || out_dtype == FW_BF16, "rglru_scan: unknown dtype %d", out_dtype);
    dim3 grid(segments, (unsigned)fw_ceil_div(channels, 64));
    hipStream_t s = (hipStream_t)stream;
    // a step that may hold a long segment brings a workspace (2 * rows * channels floats): such segments are walked in chunks
    const int long_apart = workspace != nullptr && rows > SCAN_LONG;
    if (out_dtype == FW_F32)
        rglru_scan_kernel<float><<<grid, 64, 0, s>>>(u, u_stride, gates, gates_stride, y, y_stride, r_bias, i_bias, lam, rate, state, seg_row0,
                                                     seg_slot, (float*)out, channels, block_width, long_apart);
    else
        rglru_scan_kernel<bf16_t><<<grid, 64, 0, s>>>(u, u_stride, gates, gates_stride, y, y_stride, r_bias, i_bias, lam, rate, state,
                                                      seg_row0, seg_slot, (bf16_t*)out, channels, block_width, long_apart);
    FW_LAUNCH_CHECK("rglru_scan");
    if (long_apart) {
        const int chunks = fw_ceil_div(rows, SCAN_CHUNK);
        FW_REQUIRE(chunks <= 65535 && grid.y <= 65535, "rglru_scan: too many rows or channels (%d, %d)", rows, channels);
        dim3 by_chunk(segments, grid.y, chunks);
        float* local = workspace;
        float* carry = workspace + (size_t)rows * channels;
        rglru_chunk_local_kernel<<<by_chunk, 64, 0, s>>>(u, u_stride, gates, gates_stride, r_bias, i_bias, lam, rate, state, seg_row0, seg_slot,
                                                         local, carry, channels, block_width);
        FW_LAUNCH_CHECK("rglru_scan (chunks)");
        if (out_dtype == FW_F32)
            rglru_chunk_finish_kernel<float><<<by_chunk, 64, 0, s>>>(y, y_stride, local, carry, state, seg_row0, seg_slot, (float*)out, channels);
        else
            rglru_chunk_finish_kernel<bf16_t><<<by_chunk, 64, 0, s>>>(y, y_stride, local, carry, state, seg_row0, seg_slot, (bf16_t*)out, channels);
        FW_LAUNCH_CHECK("rglru_scan (finish)");
    }
    return 0;
}
