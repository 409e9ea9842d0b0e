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

template <typename TO>
__global__ __launch_bounds__(64) void rglru_scan_kernel(
    const float* __restrict__ u, int u_stride, const float* __restrict__ gates, int gates_stride, const float* __restrict__ y,
    int y_stride, const float* __restrict__ r_bias, const float* __restrict__ i_bias, const float* __restrict__ lam, float rate,
    float* __restrict__ state, const int32_t* __restrict__ seg_row0, const int32_t* __restrict__ seg_slot, TO* __restrict__ out,
    int channels, int block_width) {
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    const int seg = blockIdx.x;
    if (c >= channels) return;
    const int first = seg_row0[seg], end = seg_row0[seg + 1];
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
            const float r = rglru_sigmoid(gr[k] + br), i = rglru_sigmoid(gi[k] + bi);
            // 1 - a^2 as -expm1(2 log a): a channel that barely forgets has a near 1, where 1 - a * a would lose its digits
            a[k] = expf(decay * r);
            b[k] = sqrtf(-expm1f(2.0f * decay * r)) * (i * uu[k]);
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
                             int channels, int block_width, int slots, void* stream) {
    FW_REQUIRE(rows >= 0 && segments >= 0 && channels > 0 && slots > 0,
               "rglru_scan: bad sizes rows=%d segments=%d channels=%d slots=%d", rows, segments, channels, slots);
    FW_REQUIRE(block_width > 0 && channels % block_width == 0, "rglru_scan: %d channels are not blocks of %d", channels, block_width);
    FW_REQUIRE(u_stride >= channels && y_stride >= channels && gates_stride >= 2 * channels,
               "rglru_scan: rows %d / %d / %d wide do not hold %d channels (and twice as many gates)", u_stride, y_stride, gates_stride, channels);
    FW_REQUIRE(rate > 0.0f, "rglru_scan: the decay's rate must be positive");
    if (rows == 0 || segments == 0) return 0;
    dim3 grid(segments, (unsigned)fw_ceil_div(channels, 64));
    hipStream_t s = (hipStream_t)stream;
    if (out_dtype == FW_F32)
        rglru_scan_kernel<float><<<grid, 64, 0, s>>>(u, u_stride, gates, gates_stride, y, y_stride, r_bias, i_bias, lam, rate, state, seg_row0,
                                                     seg_slot, (float*)out, channels, block_width);
    else if (out_dtype == FW_BF16)
        rglru_scan_kernel<bf16_t><<<grid, 64, 0, s>>>(u, u_stride, gates, gates_stride, y, y_stride, r_bias, i_bias, lam, rate, state,
                                                      seg_row0, seg_slot, (bf16_t*)out, channels, block_width);
    else
        FW_REQUIRE(false, "rglru_scan: unknown dtype %d", out_dtype);
    FW_LAUNCH_CHECK("rglru_scan");
    return 0;
}
