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
// row: it alone reads and writes the slot, each thread its own channels, the read first. A step of few rows
// has several workgroups a row (blockIdx.y), each with channels of its own (and the row's sums of squares once
// more): a single token's mixes are then a few loads deep, not one round of loads after the other.
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
    for (int i = blockIdx.y * 256 + threadIdx.x; i < hidden; i += 256 * gridDim.y) {
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
    const int parts = rows <= 128 ? (fw_ceil_div(hidden, 256) < 16 ? fw_ceil_div(hidden, 256) : 16) : 1;
    const dim3 grid(rows, parts);
    if (out_dtype == FW_F32)
        token_shift_mix_kernel<float><<<grid, 256, 0, s>>>(x, norm_weight, eps, one_centered, mu, mixes, last, row_seg, seg_row0, seg_slot,
                                                           (float*)out, rows, hidden);
    else if (out_dtype == FW_BF16)
        token_shift_mix_kernel<bf16_t><<<grid, 256, 0, s>>>(x, norm_weight, eps, one_centered, mu, mixes, last, row_seg, seg_row0, seg_slot,
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
// Workgroup (segment, head, block of 16 value channels); thread = 16 * column + part: a column of S is
// shared out over the 16 lanes of a row of the wave, RPT neighbouring key channels each (a lane reads its
// channels of r, of k and of the decay from LDS in one access each; channels from dim on hold zeros), so that a head is spread over many compute units: the walk along the tokens is one dependent
// chain per column (a single multiply-add per key channel and token), and only its width can be bought.
// Tokens come in chunks of WKV_CHUNK (32, fewer for wide heads, whose tokens are larger). A chunk's r, k, a
// and its block's 16 values travel from global
// memory into registers while the chunk before is walked; on their way into LDS the decay's two
// exponentials are taken, once per chunk and key channel. A column's sums over key channels (the read-out
// S^T r and the bonus r . (u k), which every column forms for itself) are each thread's own sum and then
// the sixteen lanes', inside the vector unit. The state is read at the segment's start and written at its
// end. Columns of S never meet and the lanes' sums have one fixed order, so the result depends neither on
// how the work is cut nor, tokens being walked in order whatever the segments, on the cut of the sequence.
#define WKV_LANES 16
#define WKV_COLUMNS (256 / WKV_LANES)
template <int CTRL>
__device__ __forceinline__ float wkv_dpp(float x) {
    return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(x), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float wkv_row_sum(float x) {
    x += wkv_dpp<0xB1>(x);          // quad_perm [1, 0, 3, 2]
    x += wkv_dpp<0x4E>(x);          // quad_perm [2, 3, 0, 1]
    x += wkv_dpp<0x141>(x);         // row_half_mirror
    x += wkv_dpp<0x140>(x);         // row_mirror
    return x;
}

template <int RPT, int WKV_CHUNK>
__global__ __launch_bounds__(256) void wkv_recurrence_kernel(
    const float* __restrict__ r, const float* __restrict__ k, const float* __restrict__ v, int rkv_stride,
    const float* __restrict__ a, int a_stride, const float* __restrict__ w0, const float* __restrict__ u, float* __restrict__ state,
    float* __restrict__ out, const int32_t* __restrict__ seg_row0, const int32_t* __restrict__ seg_slot, int heads, int dim) {
    constexpr int DP = WKV_LANES * RPT;                 // key channels as the lanes hold them
    constexpr int TOKEN = 3 * DP + WKV_COLUMNS;         // a staged token: r, k, decay, the block's values
    constexpr int PIECES = (WKV_CHUNK * DP + 255) / 256;    // elements of a chunk's r (and k, and a) per thread, at most
    __shared__ __attribute__((aligned(16))) float staged[WKV_CHUNK * TOKEN];
    __shared__ float results[WKV_CHUNK * WKV_COLUMNS];
    constexpr int VALUE_PIECES = (WKV_CHUNK * WKV_COLUMNS + 255) / 256;     // of the block's values of a chunk per thread
    const int seg = blockIdx.x, head = blockIdx.y, block = blockIdx.z;
    const int local = threadIdx.x / WKV_LANES, part = threadIdx.x % WKV_LANES;
    const int column = block * WKV_COLUMNS + local;
    const bool live = column < dim;
    const int first = seg_row0[seg], count = seg_row0[seg + 1] - first;
    const size_t head_at = (size_t)head * dim;
    // This thread's elements of every chunk: element e = thread + 256 i of the chunk's [tokens][dim] block of r,
    // of k and of a alike (token e / dim, channel e % dim), and one of the block's values (token thread / 16,
    // column thread % 16). A token of -1: no such element.
    int piece_token[PIECES], piece_channel[PIECES];
    float piece_w0[PIECES];
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
        const int e = threadIdx.x + 256 * i;
        const bool there = e < WKV_CHUNK * dim;
        piece_token[i] = there ? e / dim : -1;
        piece_channel[i] = there ? e % dim : 0;
        piece_w0[i] = w0[head_at + piece_channel[i]];
    }
    const int value_column = block * WKV_COLUMNS + threadIdx.x % WKV_COLUMNS;
    int value_token[VALUE_PIECES];
#pragma unroll
    for (int j = 0; j < VALUE_PIECES; ++j) {
        const int token = (threadIdx.x + 256 * j) / WKV_COLUMNS;
        value_token[j] = (token < WKV_CHUNK && value_column < dim) ? token : -1;
    }
    const int staged_tokens = count < WKV_CHUNK ? count : WKV_CHUNK;        // a decode step stages one token
    for (int i = threadIdx.x; i < staged_tokens * TOKEN; i += 256) staged[i] = 0.0f;
    float held_r[PIECES], held_k[PIECES], held_a[PIECES], held_v[VALUE_PIECES];
    // Loads are unconditional and their addresses plain arithmetic (an element past the chunk's end, or one that
    // this thread does not have, is read from a valid place again and never used): behind a branch the compiler
    // would wait for each load at once, and the next chunk would not travel while this one is walked.
    auto ask = [&](int base) {
        const int last = (count - base < WKV_CHUNK ? count - base : WKV_CHUNK) - 1;
        const float* r0 = r + (size_t)(first + base) * rkv_stride + head_at;
        const float* k0 = k + (size_t)(first + base) * rkv_stride + head_at;
        const float* v0 = v + (size_t)(first + base) * rkv_stride + head_at;
        const float* a0 = a + (size_t)(first + base) * a_stride + head_at;
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            int token = piece_token[i] < 0 ? 0 : piece_token[i];
            token = token < last ? token : last;
            held_r[i] = r0[token * rkv_stride + piece_channel[i]];
            held_k[i] = k0[token * rkv_stride + piece_channel[i]];
            held_a[i] = a0[token * a_stride + piece_channel[i]];
        }
#pragma unroll
        for (int j = 0; j < VALUE_PIECES; ++j) {
            int token = value_token[j] < 0 ? 0 : value_token[j];
            token = token < last ? token : last;
            held_v[j] = v0[token * rkv_stride + (value_token[j] < 0 ? 0 : value_column)];
        }
    };
    auto put = [&](int base) {
        const int tokens = count - base < WKV_CHUNK ? count - base : WKV_CHUNK;
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const float decay = expf(-expf(held_a[i] + piece_w0[i]));
            if (piece_token[i] >= 0 && piece_token[i] < tokens) {
                float* to = staged + piece_token[i] * TOKEN + piece_channel[i];
                to[0] = held_r[i];
                to[DP] = held_k[i];
                to[2 * DP] = decay;
            }
        }
#pragma unroll
        for (int j = 0; j < VALUE_PIECES; ++j)
            if (value_token[j] >= 0 && value_token[j] < tokens) staged[value_token[j] * TOKEN + 3 * DP + threadIdx.x % WKV_COLUMNS] = held_v[j];
    };
    ask(0);
    float* mine = state + ((size_t)seg_slot[seg] * heads + head) * dim * dim + (live ? column : 0);
    float S[RPT], bonus[RPT];
#pragma unroll
    for (int t = 0; t < RPT; ++t) {
        const int key = part * RPT + t;
        S[t] = (live && key < dim) ? mine[(size_t)key * dim] : 0.0f;
        bonus[t] = key < dim ? u[head_at + key] : 0.0f;
    }
    __syncthreads();        // the zeros are in place
    put(0);
    __syncthreads();
    for (int base = 0; base < count; base += WKV_CHUNK) {
        const int tokens = count - base < WKV_CHUNK ? count - base : WKV_CHUNK;
        const bool more = base + WKV_CHUNK < count;
        if (more) ask(base + WKV_CHUNK);
        // a token's operands are read from LDS while the token before it is worked on
        float r_next[RPT], k_next[RPT], w_next[RPT], v_next;
        auto fetch = [&](int token) {
            const float* t0 = staged + token * TOKEN;
#pragma unroll
            for (int t = 0; t < RPT; ++t) {
                r_next[t] = t0[part * RPT + t];
                k_next[t] = t0[DP + part * RPT + t];
                w_next[t] = t0[2 * DP + part * RPT + t];
            }
            v_next = t0[3 * DP + local];
        };
        fetch(0);
        for (int token = 0; token < tokens; ++token) {
            const float value = v_next;
            float read = 0.0f, ruk = 0.0f;
#pragma unroll
            for (int t = 0; t < RPT; ++t) {
                read = fmaf(r_next[t], S[t], read);
                ruk = fmaf(r_next[t] * bonus[t], k_next[t], ruk);
                S[t] = fmaf(w_next[t], S[t], k_next[t] * value);
            }
            fetch(token + 1 < staged_tokens ? token + 1 : token);       // (behind the chunk's last token: read again, not used)
            read = wkv_row_sum(read);
            ruk = wkv_row_sum(ruk);
            if (part == 0) results[token * WKV_COLUMNS + local] = fmaf(ruk, value, read);
        }
        // (barriers that order LDS traffic only: the next chunk's loads stay in flight across them)
        fw_lds_barrier();
        // the chunk's read-outs leave together: a token's 16 columns side by side
        for (int i = threadIdx.x; i < tokens * WKV_COLUMNS; i += 256) {
            const int token = i / WKV_COLUMNS, c = i % WKV_COLUMNS;
            if (block * WKV_COLUMNS + c < dim)
                out[((size_t)first + base + token) * heads * dim + head_at + block * WKV_COLUMNS + c] = results[i];
        }
        if (more) put(base + WKV_CHUNK);
        fw_lds_barrier();
    }
    if (live) {
#pragma unroll
        for (int t = 0; t < RPT; ++t) {
            const int key = part * RPT + t;
            if (key < dim) mine[(size_t)key * dim] = S[t];
        }
    }
}

extern "C" int fw_wkv_recurrence(const float* r, const float* k, const float* v, int rkv_stride, const float* a, int a_stride,
                                 const float* w0, const float* u, float* state, int slots, float* out, const int32_t* seg_row0,
                                 const int32_t* seg_slot, int rows, int segments, int heads, int dim, void* stream) {
    FW_REQUIRE(rows >= 0 && segments >= 0 && heads > 0 && heads <= 65535 && slots > 0, "wkv_recurrence: bad sizes rows=%d segments=%d heads=%d", rows, segments, heads);
    FW_REQUIRE(dim >= 1 && dim <= 256, "wkv_recurrence: a head of %d channels (1..256)", dim);
    FW_REQUIRE(rkv_stride >= heads * dim && a_stride >= heads * dim, "wkv_recurrence: rows of %d / %d values do not hold %d heads of %d", rkv_stride, a_stride, heads, dim);
    if (rows == 0 || segments == 0) return 0;
    dim3 grid(segments, heads, (dim + WKV_COLUMNS - 1) / WKV_COLUMNS);
    hipStream_t s = (hipStream_t)stream;
#define FW_WKV_LAUNCH(RPT, CHUNK) \
    wkv_recurrence_kernel<RPT, CHUNK><<<grid, 256, 0, s>>>(r, k, v, rkv_stride, a, a_stride, w0, u, state, out, seg_row0, seg_slot, heads, dim)
    // (the chunk's length changes what is staged together, not one sum: steps of single tokens take short chunks,
    // whose bookkeeping at the start is a few loads)
    const bool few = rows <= 4 * segments;
    if (dim <= 16) { if (few) FW_WKV_LAUNCH(1, 4); else FW_WKV_LAUNCH(1, 32); }
    else if (dim <= 32) { if (few) FW_WKV_LAUNCH(2, 4); else FW_WKV_LAUNCH(2, 32); }
    else if (dim <= 64) { if (few) FW_WKV_LAUNCH(4, 4); else FW_WKV_LAUNCH(4, 32); }
    else if (dim <= 128) FW_WKV_LAUNCH(8, 8);
    else FW_WKV_LAUNCH(16, 4);
#undef FW_WKV_LAUNCH
    FW_LAUNCH_CHECK("wkv_recurrence");
    return 0;
}
