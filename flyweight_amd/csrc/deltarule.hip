// The gated delta rule: a linear recurrence over a matrix state per head, with the short causal
// convolutions in front of it and the gated norm behind it. Everything here is float32.
//
// Per head, with state S [dim][vdim], a token brings a query q and key k (dim channels, unit vectors),
// a value v (vdim channels), a write strength beta and a decay g per key channel:
//     S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// so the read-out sees the token's own write. Columns of S (value channels) never meet: a column is
// owned by sixteen lanes, each holding a sixteenth of its rows in registers, and the two sums over the
// key channels are reductions over those lanes. A segment's tokens are walked in order. What a
// token brings to a head lies in one record, [q | k | g | beta | v] (fw_delta_record_floats), so that a
// chunk of tokens is a plain copy into LDS; the copy of the next chunk is asked for before the work on
// this one and waits in registers meanwhile.
//
// The state is stored transposed, [slot][head][vdim][dim], so that the columns a wave holds are one
// contiguous piece of memory.
#include "fw_common.h"
#include "fw_kernels.h"

#define DELTA_CHUNK 16          // tokens staged in LDS at a time

__device__ __forceinline__ float fw_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float fw_softplus(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

// ---- what the recurrence reads, from the projections -----------------------------------------------
// One wave per (row, vector). Vectors 0..G-1: query heads, G..2G-1: key heads (dim channels each,
// convolution, silu, then unit length; queries also times dim^-1/2); then H value heads (vdim
// channels, convolution and silu); then H decay vectors (dim channels, no convolution):
// g = exp(-exp(A_log[h]) * softplus(a + dt_bias)); lane 0 of a decay vector also forms beta.
// proj [rows][proj_stride]: columns 0.. hold q | k | v (the convolution's inputs), column beta_col + h
// the write strength before its sigmoid. state [slots][C][L-1]: the inputs of the L-1 tokens before
// the segment, oldest first. The state is read here and moved on by conv_state_kernel afterwards;
// with SINGLE (every segment is one row: a decode step) the wave that read a channel's memory moves it
// on itself. a [rows][a_stride]: the decays' arguments in its first heads * dim columns.
template <typename TI, bool SINGLE>
__global__ __launch_bounds__(64) void delta_prepare_kernel(
    const TI* __restrict__ proj, int proj_stride, int beta_col, const TI* __restrict__ a, int a_stride, const float* __restrict__ taps,
    float* __restrict__ conv_state, const float* __restrict__ A_log, const float* __restrict__ dt_bias,
    const int32_t* __restrict__ row_seg, const int32_t* __restrict__ seg_row0, const int32_t* __restrict__ seg_slot,
    float* __restrict__ records, int heads, int kv_heads, int dim, int vdim, int taps_count, int decay_per_head) {
    const int row = blockIdx.x, vec = blockIdx.y, lane = threadIdx.x;
    const int conv_channels = 2 * kv_heads * dim + heads * vdim;
    const int d4 = (dim + 3) & ~3, v4 = (vdim + 3) & ~3;
    const int record = 3 * d4 + 4 + v4;                     // q | k | g | beta and three unused | v
    float* of_row = records + (size_t)row * heads * record;
    if (vec >= 2 * kv_heads + heads) {      // a decay vector
        const int h = vec - 2 * kv_heads - heads;
        const float rate = expf(A_log[h]);
        float* dest = of_row + (size_t)h * record + 2 * d4;
        for (int i = lane; i < d4; i += 64) {
            const int at = decay_per_head ? h : h * dim + i;    // one decay for the head: every key channel gets it
            dest[i] = i < dim ? expf(-rate * fw_softplus(load_as_float(a, (size_t)row * a_stride + at) + dt_bias[at])) : 0.0f;
        }
        if (lane < 4) dest[d4 + lane] = lane == 0 ? fw_sigmoid(load_as_float(proj, (size_t)row * proj_stride + beta_col + h)) : 0.0f;
        return;
    }
    const bool value = vec >= 2 * kv_heads;
    const int width = value ? vdim : dim;
    const int c0 = value ? 2 * kv_heads * dim + (vec - 2 * kv_heads) * vdim : vec * dim;
    const int seg = row_seg[row];
    const int first = seg_row0[seg];
    float* before = conv_state + (size_t)seg_slot[seg] * conv_channels * (taps_count - 1);
    float sum_sq = 0.0f;
    // a vector of up to 256 channels: four per lane
    float kept[4];
#pragma unroll
    for (int part = 0; part < 4; ++part) {
        const int i = lane + 64 * part;
        float y = 0.0f;
        if (i < width) {
            const int c = c0 + i;
            float acc = 0.0f;
            for (int j = 0; j < taps_count; ++j) {
                const int back = taps_count - 1 - j;        // tap j looks this many tokens back
                const int r = row - back;
                const float x = r >= first ? load_as_float(proj, (size_t)r * proj_stride + c)
                                           : before[(size_t)c * (taps_count - 1) + (taps_count - 1 + (r - first))];
                acc = fmaf(taps[(size_t)c * taps_count + j], x, acc);
                // the memory moves on by this row: entry j - 1 takes x, and no later tap reads it
                if (SINGLE && j > 0) before[(size_t)c * (taps_count - 1) + j - 1] = x;
            }
            y = acc * fw_sigmoid(acc);
        }
        kept[part] = y;
        sum_sq += y * y;
    }
    float factor = 1.0f;
    if (!value) {
        sum_sq = wave_sum(sum_sq);
        factor = 1.0f / sqrtf(sum_sq + 1e-6f);
        if (vec < kv_heads) factor *= 1.0f / sqrtf((float)dim);
    }
    // a value head goes to its head's record; a query or key head to the records of every head of its group
    const int group = heads / kv_heads;
    const int first_head = value ? vec - 2 * kv_heads : (vec % kv_heads) * group;
    const int copies = value ? 1 : group;
    const int at = value ? 3 * d4 + 4 : (vec < kv_heads ? 0 : d4);
    const int padded = value ? v4 : d4;
    for (int copy = 0; copy < copies; ++copy) {
        float* dest = of_row + (size_t)(first_head + copy) * record + at;
#pragma unroll
        for (int part = 0; part < 4; ++part) {
            const int i = lane + 64 * part;
            if (i < padded) dest[i] = i < width ? kept[part] * factor : 0.0f;
        }
    }
}

// The convolution's memory moves on: a thread per (segment, channel) reads the L-1 old inputs, then
// writes the last L-1 of (old inputs, the segment's inputs).
template <typename TI>
__global__ void conv_state_kernel(const TI* __restrict__ proj, int proj_stride, float* __restrict__ conv_state,
                                  const int32_t* __restrict__ seg_row0, const int32_t* __restrict__ seg_slot,
                                  int channels, int taps_count) {
    const int seg = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int first = seg_row0[seg], count = seg_row0[seg + 1] - first;
    const int keep = taps_count - 1;
    float* state = conv_state + ((size_t)seg_slot[seg] * channels + c) * keep;
    float old[16];
    for (int i = 0; i < keep; ++i) old[i] = state[i];
    for (int i = 0; i < keep; ++i) {
        const int at = count - keep + i;        // place among the segment's rows; negative: among the old inputs
        state[i] = at >= 0 ? load_as_float(proj, (size_t)(first + at) * proj_stride + c) : old[keep + at];
    }
}

extern "C" int fw_delta_prepare(const void* proj, int dtype, int proj_stride, int beta_col, const void* a, int a_stride, const float* taps,
                                float* conv_state, const float* A_log, const float* dt_bias, const int32_t* row_seg,
                                const int32_t* seg_row0, const int32_t* seg_slot, float* records, int rows, int segments,
                                int heads, int kv_heads, int dim, int vdim, int taps_count, int slots, int decay_per_head,
                                void* stream) {
    FW_REQUIRE(rows >= 0 && segments >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
               "delta_prepare: heads %d must be a positive multiple of kv heads %d", heads, kv_heads);
    FW_REQUIRE(dim > 0 && dim <= 256 && vdim > 0 && vdim <= 256, "delta_prepare: dim %d and vdim %d must lie in 1..256", dim, vdim);
    FW_REQUIRE(taps_count >= 1 && taps_count <= 17, "delta_prepare: %d taps outside 1..17", taps_count);
    FW_REQUIRE(slots > 0, "delta_prepare: no state slots");
    const int channels = 2 * kv_heads * dim + heads * vdim;
    FW_REQUIRE(proj_stride >= channels && beta_col >= 0 && beta_col + heads <= proj_stride,
               "delta_prepare: the projections' rows (%d wide) do not hold %d channels and %d strengths at %d", proj_stride, channels, heads, beta_col);
    FW_REQUIRE(a_stride >= (decay_per_head ? heads : heads * dim), "delta_prepare: the decays' arguments (%d wide) do not hold %d x %d", a_stride, heads, decay_per_head ? 1 : dim);
    FW_REQUIRE(rows <= 1 << 20 && segments <= 65535 && 2 * kv_heads + 2 * heads <= 65535, "delta_prepare: too many rows, segments or heads");
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(rows, 2 * kv_heads + 2 * heads);
    dim3 state_grid((channels + 127) / 128, segments);
    const bool single = rows == segments;       // every segment one row: the memory moves on inside the one kernel
#define FW_PREPARE_LAUNCH(TI, SINGLE)                                                                                         \
    delta_prepare_kernel<TI, SINGLE><<<grid, 64, 0, s>>>((const TI*)proj, proj_stride, beta_col, (const TI*)a, a_stride, taps, \
                                                         conv_state, A_log, dt_bias, row_seg, seg_row0, seg_slot, records,     \
                                                         heads, kv_heads, dim, vdim, taps_count, decay_per_head)
    if (dtype == FW_F32) {
        if (single) FW_PREPARE_LAUNCH(float, true);
        else FW_PREPARE_LAUNCH(float, false);
        if (taps_count > 1 && !single)
            conv_state_kernel<float><<<state_grid, 128, 0, s>>>((const float*)proj, proj_stride, conv_state, seg_row0, seg_slot, channels, taps_count);
    } else if (dtype == FW_BF16) {
        if (single) FW_PREPARE_LAUNCH(bf16_t, true);
        else FW_PREPARE_LAUNCH(bf16_t, false);
        if (taps_count > 1 && !single)
            conv_state_kernel<bf16_t><<<state_grid, 128, 0, s>>>((const bf16_t*)proj, proj_stride, conv_state, seg_row0, seg_slot, channels, taps_count);
    } else {
        FW_REQUIRE(false, "delta_prepare: unknown dtype %d", dtype);
    }
#undef FW_PREPARE_LAUNCH
    FW_LAUNCH_CHECK("delta_prepare");
    return 0;
}

// ---- the recurrence -----------------------------------------------------------------------------
extern "C" int fw_delta_record_floats(int dim, int vdim) { return 3 * ((dim + 3) & ~3) + 4 + ((vdim + 3) & ~3); }

// A sum over the 16 lanes of a row of the wave (every lane gets it): neighbours, pairs, then the two
// mirrors, all inside the vector unit (no trip through the LDS crossbar). After each step the lanes
// that have met hold one value, so the mirrors may stand for the exchanges between quads and halves.
template <int CTRL>
__device__ __forceinline__ float delta_dpp(float x) {
    return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(x), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float delta_row_sum(float x) {
    x += delta_dpp<0xB1>(x);        // quad_perm [1, 0, 3, 2]
    x += delta_dpp<0x4E>(x);        // quad_perm [2, 3, 0, 1]
    x += delta_dpp<0x141>(x);       // row_half_mirror
    x += delta_dpp<0x140>(x);       // row_mirror
    return x;
}

// Workgroup (segment, head, block of 16 value channels); thread = 16 * column + part: a column of S
// is shared out over the 16 lanes of a row of the wave, RPT rows each (rows part, part + 16, ...: the
// sixteen lanes then read sixteen neighbouring floats of q, k and g from LDS, one bank each; rows from
// dim on hold zeros), so that a head is spread over many compute units: the walk along the
// tokens is one dependent chain per column, and only its width can be bought. LDS per staged token:
// q, k, g (16 * RPT each; past the record's padded dim they stay zero), beta and three unused, then the
// block's 16 values. A thread copies the same pieces of every chunk (16-byte pieces: where each lies in
// a token's record and in LDS is worked out once).
#define DELTA_LANES 16
#define DELTA_COLUMNS (256 / DELTA_LANES)
template <int RPT>
__global__ __launch_bounds__(256) void gated_delta_rule_kernel(
    const float* __restrict__ records, float* __restrict__ state, float* __restrict__ out,
    const int32_t* __restrict__ seg_row0, const int32_t* __restrict__ seg_slot, int heads, int dim, int vdim) {
    typedef __attribute__((ext_vector_type(4))) float f32x4;
    constexpr int DP = DELTA_LANES * RPT;
    constexpr int TOKEN = 3 * DP + 4 + DELTA_COLUMNS;
    constexpr int PIECES = (DELTA_CHUNK * (TOKEN / 4) + 255) / 256;      // 16-byte pieces of a chunk per thread, at most
    __shared__ __attribute__((aligned(16))) float staged[DELTA_CHUNK * TOKEN];
    __shared__ float results[DELTA_CHUNK * DELTA_COLUMNS];
    static_assert(DELTA_CHUNK * DELTA_COLUMNS == 256, "a chunk's read-outs are one per thread");
    const int seg = blockIdx.x, head = blockIdx.y, block = blockIdx.z;
    const int local = threadIdx.x / DELTA_LANES, part = threadIdx.x % DELTA_LANES;
    const int column = block * DELTA_COLUMNS + local;
    const bool live = column < vdim;
    const int first = seg_row0[seg], count = seg_row0[seg + 1] - first;
    const int d4 = (dim + 3) & ~3, v4 = (vdim + 3) & ~3;
    const int record = 3 * d4 + 4 + v4;
    const int values_here = v4 - block * DELTA_COLUMNS < DELTA_COLUMNS ? v4 - block * DELTA_COLUMNS : DELTA_COLUMNS;
    const int per_token = (3 * d4 + 4 + values_here) / 4;                // pieces of a token that this block needs
    // this thread's pieces: token of the chunk, place in the record, place in LDS
    int piece_token[PIECES], piece_from[PIECES], piece_to[PIECES];
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
        const int item = threadIdx.x + 256 * i;
        const int token = item / per_token, f = (item % per_token) * 4;
        piece_token[i] = token < DELTA_CHUNK ? token : DELTA_CHUNK;       // DELTA_CHUNK: this thread has no such piece
        int from, to;
        if (f < 3 * d4) {
            from = f;
            to = (f / d4) * DP + f % d4;
        } else if (f == 3 * d4) {
            from = f;
            to = 3 * DP;
        } else {
            from = 3 * d4 + 4 + block * DELTA_COLUMNS + (f - 3 * d4 - 4);
            to = 3 * DP + 4 + (f - 3 * d4 - 4);
        }
        piece_from[i] = token < DELTA_CHUNK ? from : 0;
        piece_to[i] = (token < DELTA_CHUNK ? token : 0) * TOKEN + to;
    }
    const int staged_tokens = count < DELTA_CHUNK ? count : DELTA_CHUNK;     // a decode step stages one token
    for (int i = threadIdx.x; i < staged_tokens * TOKEN; i += 256) staged[i] = 0.0f;
    const float* source = records + ((size_t)first * heads + head) * record;
    const size_t token_stride = (size_t)heads * record;
    f32x4 held[PIECES];
    // Loads are unconditional (a piece past the chunk's end is read from a valid place again and never
    // used): behind a branch the compiler would wait for each load at once, and the next chunk would
    // not travel while this one is worked on.
    auto ask = [&](int base) {
        const int last = (count - base < DELTA_CHUNK ? count - base : DELTA_CHUNK) - 1;
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int token = piece_token[i] < last ? piece_token[i] : last;
            held[i] = *reinterpret_cast<const f32x4*>(source + (size_t)(base + token) * token_stride + piece_from[i]);
        }
    };
    auto put = [&](int base) {
        const int tokens = count - base < DELTA_CHUNK ? count - base : DELTA_CHUNK;
#pragma unroll
        for (int i = 0; i < PIECES; ++i)
            if (piece_token[i] < tokens) *reinterpret_cast<f32x4*>(staged + piece_to[i]) = held[i];
    };
    ask(0);
    float* mine = state + (((size_t)seg_slot[seg] * heads + head) * vdim + (live ? column : 0)) * dim;
    float S[RPT];
#pragma unroll
    for (int t = 0; t < RPT; ++t) {
        const int i = t * DELTA_LANES + part;
        S[t] = (live && i < dim) ? mine[i] : 0.0f;
    }
    __syncthreads();        // the zeros are in place
    put(0);
    __syncthreads();
    for (int base = 0; base < count; base += DELTA_CHUNK) {
        const int tokens = count - base < DELTA_CHUNK ? count - base : DELTA_CHUNK;
        const bool more = base + DELTA_CHUNK < count;
        if (more) ask(base + DELTA_CHUNK);
        // a token's operands are read from LDS while the token before it is worked on
        float q_next[RPT], k_next[RPT], g_next[RPT], b_next, v_next;
        auto fetch = [&](int token) {
            const float* t0 = staged + token * TOKEN;
#pragma unroll
            for (int t = 0; t < RPT; ++t) {
                q_next[t] = t0[t * DELTA_LANES + part];
                k_next[t] = t0[DP + t * DELTA_LANES + part];
                g_next[t] = t0[2 * DP + t * DELTA_LANES + part];
            }
            b_next = t0[3 * DP];
            v_next = t0[3 * DP + 4 + local];
        };
        fetch(0);
        for (int token = 0; token < tokens; ++token) {
            // The chain from token to token is: decay, the sum over key channels, the write. The read-out
            // o = (S' + k u^T)^T q = S'^T q + u (k . q) with S' = diag(g) S is formed beside it from sums
            // that do not wait for u: all three sums of a token travel through the lanes together.
            float k_now[RPT];
            const float b = b_next, v = v_next;
            float seen = 0.0f, read_before = 0.0f, kq = 0.0f;
#pragma unroll
            for (int t = 0; t < RPT; ++t) {
                k_now[t] = k_next[t];
                S[t] *= g_next[t];
                seen = fmaf(S[t], k_now[t], seen);
                read_before = fmaf(S[t], q_next[t], read_before);
                kq = fmaf(k_now[t], q_next[t], kq);
            }
            fetch(token + 1 < DELTA_CHUNK ? token + 1 : token);      // (behind the chunk's last token: read again, not used)
            seen = delta_row_sum(seen);
            read_before = delta_row_sum(read_before);
            kq = delta_row_sum(kq);
            const float u = b * (v - seen);
#pragma unroll
            for (int t = 0; t < RPT; ++t) S[t] = fmaf(k_now[t], u, S[t]);
            if (part == 0) results[token * DELTA_COLUMNS + local] = fmaf(u, kq, read_before);
        }
        // (barriers that order LDS traffic only: the next chunk's loads stay in flight across them)
        fw_lds_barrier();
        // the chunk's read-outs leave together: a token's 16 columns side by side
        {
            const int token = threadIdx.x / DELTA_COLUMNS, c = threadIdx.x % DELTA_COLUMNS;
            if (token < tokens && block * DELTA_COLUMNS + c < vdim)
                out[((size_t)first + base + token) * heads * vdim + head * vdim + block * DELTA_COLUMNS + c] = results[threadIdx.x];
        }
        if (more) put(base + DELTA_CHUNK);
        fw_lds_barrier();
    }
    if (live) {
#pragma unroll
        for (int t = 0; t < RPT; ++t) {
            const int i = t * DELTA_LANES + part;
            if (i < dim) mine[i] = S[t];
        }
    }
}

extern "C" int fw_gated_delta_rule(const float* records, float* state, float* out, const int32_t* seg_row0,
                                   const int32_t* seg_slot, int rows, int segments, int heads, int dim, int vdim,
                                   int slots, void* stream) {
    FW_REQUIRE(rows >= 0 && segments >= 0 && heads > 0, "gated_delta_rule: bad sizes rows=%d segments=%d heads=%d", rows, segments, heads);
    FW_REQUIRE(dim > 0 && dim <= 256 && vdim > 0, "gated_delta_rule: dim %d must lie in 1..256 and vdim %d be positive", dim, vdim);
    FW_REQUIRE(slots > 0 && segments <= 65535 && heads <= 65535, "gated_delta_rule: too many segments or heads, or no slots");
    FW_REQUIRE((uintptr_t)records % 16 == 0, "gated_delta_rule: the records must lie at a multiple of 16 bytes");
    if (rows == 0 || segments == 0) return 0;
    dim3 grid(segments, heads, (vdim + DELTA_COLUMNS - 1) / DELTA_COLUMNS);
    hipStream_t s = (hipStream_t)stream;
#define FW_DELTA_LAUNCH(RPT) \
    gated_delta_rule_kernel<RPT><<<grid, 256, 0, s>>>(records, state, out, seg_row0, seg_slot, heads, dim, vdim)
    if (dim <= 16) FW_DELTA_LAUNCH(1);
    else if (dim <= 32) FW_DELTA_LAUNCH(2);
    else if (dim <= 64) FW_DELTA_LAUNCH(4);
    else if (dim <= 128) FW_DELTA_LAUNCH(8);
    else FW_DELTA_LAUNCH(16);
#undef FW_DELTA_LAUNCH
    FW_LAUNCH_CHECK("gated_delta_rule");
    return 0;
}

// ---- behind the recurrence: per-head RMS norm, a weight, a sigmoid gate ------------------------------
// out[r][h][j] = o[r][h][j] * rsqrt(mean_j o^2 + eps) * weight[j] * sigmoid(gate[r][gate_col + h vdim + j])
template <typename TG, typename T>
__global__ __launch_bounds__(64) void gated_head_norm_kernel(const float* __restrict__ o, const TG* __restrict__ gate, int gate_stride,
                                                            const float* __restrict__ weight, T* __restrict__ out,
                                                            int heads, int vdim, float eps, int gate_silu, int weight_per_head) {
    const int row = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const float* source = o + ((size_t)row * heads + head) * vdim;
    float sum = 0.0f;
    for (int j = lane; j < vdim; j += 64) sum += source[j] * source[j];
    sum = wave_sum(sum);
    const float inv = 1.0f / sqrtf(sum / (float)vdim + eps);
    if (weight_per_head) weight += (size_t)head * vdim;       // every head has a weight of its own, [heads][vdim]
    for (int j = lane; j < vdim; j += 64) {
        const float z = load_as_float(gate, (size_t)row * gate_stride + head * vdim + j);
        const float g = gate_silu ? z * fw_sigmoid(z) : fw_sigmoid(z);
        store_from_float(out, ((size_t)row * heads + head) * vdim + j, source[j] * inv * weight[j] * g);
    }
}

extern "C" int fw_gated_head_norm(const float* o, const void* gate, int gate_dtype, int gate_stride, const float* weight,
                                  int weight_per_head, void* out, int out_dtype, int rows, int heads, int vdim, float eps, int gate_silu, void* stream) {
    FW_REQUIRE(rows >= 0 && heads > 0 && heads <= 65535 && vdim > 0, "gated_head_norm: bad sizes rows=%d heads=%d vdim=%d", rows, heads, vdim);
    FW_REQUIRE(gate_stride >= heads * vdim, "gated_head_norm: the gates' rows (%d wide) do not hold %d x %d", gate_stride, heads, vdim);
    if (rows == 0) return 0;
    dim3 grid(rows, heads);
    hipStream_t s = (hipStream_t)stream;
#define FW_GHN_LAUNCH(TG, T) \
    gated_head_norm_kernel<TG, T><<<grid, 64, 0, s>>>(o, (const TG*)gate, gate_stride, weight, (T*)out, heads, vdim, eps, gate_silu, weight_per_head)
    if (gate_dtype == FW_F32 && out_dtype == FW_F32) FW_GHN_LAUNCH(float, float);
    else if (gate_dtype == FW_F32 && out_dtype == FW_BF16) FW_GHN_LAUNCH(float, bf16_t);
    else if (gate_dtype == FW_BF16 && out_dtype == FW_BF16) FW_GHN_LAUNCH(bf16_t, bf16_t);
    else FW_REQUIRE(false, "gated_head_norm: unsupported dtypes gate=%d out=%d", gate_dtype, out_dtype);
#undef FW_GHN_LAUNCH
    FW_LAUNCH_CHECK("gated_head_norm");
    return 0;
}
