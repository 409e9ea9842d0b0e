// Attention over a cached latent: keys and values of every head are linear maps of one normed
// vector c per token (k_h = U_h c, v_h = V_h c), so only c is cached and the maps move to the
// query's side: score = q_h . (U_h c) = (U_h^T q_h) . c, and the head's output V_h (sum_j p_j c_j).
// The attention kernels then see one shared key/value head of the latent's size. Here: the norm of
// the latent with its store into the pages, and the per-head maps on the query's and the output's side.
#include "fw_common.h"
#include "fw_kernels.h"

#define LATENT_PAGE 64

// ---- the latent of a step's rows, normed and stored ---------------------------------------------------
// raw [rows][raw_stride] float32 holds the latent before its norm in columns col0 .. col0 + rank - 1.
// c = raw / sqrt(mean(raw^2) + eps) * weight goes to both layouts of the cache's one head:
// k_pages [page][1][64][rank + rot] (a token's channels together) and v_pages [page][1][rank][64].
// rot > 0: the next rot columns of raw are a key part of the token's own that every head shares; it is not
// normed, neighbouring channels (2i, 2i + 1) of its first `turn` turn by the row's angles (tables [rows][turn / 2]), and
// it is stored behind the latent in the key layout only (a key has rank + rot channels, a value rank).
template <typename T>
__global__ __launch_bounds__(256) void latent_norm_write_kernel(
    const float* __restrict__ raw, int raw_stride, int col0, const float* __restrict__ weight, float eps,
    T* __restrict__ k_pages, T* __restrict__ v_pages, const int32_t* __restrict__ block_table, int table_stride,
    const int32_t* __restrict__ row_seg, const int32_t* __restrict__ row_pos, int rank, int rot, int turn,
    const float* __restrict__ cos_table, const float* __restrict__ sin_table) {
    __shared__ float scratch[16];
    const int row = blockIdx.x;
    const float* source = raw + (size_t)row * raw_stride + col0;
    const int pos = row_pos[row];
    const int page = block_table[(size_t)row_seg[row] * table_stride + pos / LATENT_PAGE];
    const int slot = pos % LATENT_PAGE;
    float sum = 0.0f;
    for (int j = threadIdx.x; j < rank; j += 256) sum = fmaf(source[j], source[j], sum);
    const float inv = 1.0f / sqrtf(block_sum(sum, scratch) / (float)rank + eps);
    T* key = k_pages + ((size_t)page * LATENT_PAGE + slot) * (rank + rot);
    T* value = v_pages + (size_t)page * rank * LATENT_PAGE + slot;
    for (int j = threadIdx.x; j < rank; j += 256) {
        const float c = source[j] * inv * weight[j];
        store_from_float(key, j, c);
        store_from_float(value, (size_t)j * LATENT_PAGE, c);
    }
    for (int j = threadIdx.x; j < rot; j += 256) {
        const float mine = source[rank + j];
        if (j >= turn) {        // past the turned channels: as it is
            store_from_float(key, rank + j, mine);
            continue;
        }
        const float other = source[rank + (j ^ 1)];
        const float c = cos_table[(size_t)row * (turn / 2) + (j >> 1)], sn = sin_table[(size_t)row * (turn / 2) + (j >> 1)];
        // one rounding of other * sin, then one fused step: the same in every kernel that rotates
        store_from_float(key, rank + j, fmaf(mine, c, (j & 1) ? other * sn : -(other * sn)));
    }
}

extern "C" int fw_latent_norm_write(const float* raw, int raw_stride, int col0, const float* weight, float eps, void* k_pages,
                                    void* v_pages, int dtype, const int32_t* block_table, int table_stride,
                                    const int32_t* row_seg, const int32_t* row_pos, int rows, int rank, int rot, int turn,
                                    const float* cos_table, const float* sin_table, int page_size, int num_pages, void* stream) {
    FW_REQUIRE(rows >= 0 && rank > 0 && col0 >= 0 && rot >= 0 && col0 + rank + rot <= raw_stride, "latent_norm_write: columns %d..%d of rows %d wide", col0,
               col0 + rank + rot, raw_stride);
    FW_REQUIRE(turn >= 0 && turn <= rot && turn % 2 == 0 && (turn == 0 || (cos_table && sin_table)),
               "latent_norm_write: %d turned channels of a part of %d need an even number and their tables", turn, rot);
    FW_REQUIRE(eps > 0.0f, "latent_norm_write: eps must be positive");
    FW_REQUIRE(page_size == LATENT_PAGE, "latent_norm_write: page size must be %d, got %d", LATENT_PAGE, page_size);
    FW_REQUIRE(num_pages > 0 && table_stride > 0, "latent_norm_write: empty cache (pages=%d, table stride=%d)", num_pages, table_stride);
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == FW_F32)
        latent_norm_write_kernel<float><<<rows, 256, 0, s>>>(raw, raw_stride, col0, weight, eps, (float*)k_pages, (float*)v_pages,
                                                             block_table, table_stride, row_seg, row_pos, rank, rot, turn, cos_table, sin_table);
    else if (dtype == FW_BF16)
        latent_norm_write_kernel<bf16_t><<<rows, 256, 0, s>>>(raw, raw_stride, col0, weight, eps, (bf16_t*)k_pages, (bf16_t*)v_pages,
                                                              block_table, table_stride, row_seg, row_pos, rank, rot, turn, cos_table, sin_table);
    else
        FW_REQUIRE(false, "latent_norm_write: unknown dtype %d", dtype);
    FW_LAUNCH_CHECK("latent_norm_write");
    return 0;
}

// ---- a map per head ------------------------------------------------------------------------------------
// out[r][h N + n] = sum_k in[r][h K + k] * w[h][n][k], then with a gate (float32) times sigmoid(gate[r][h N + n]).
// in [rows][in_stride], w [heads][N][K], out [rows][heads N]. A head's inputs may lie in_head apart (K of them used) and
// its outputs out_head apart in rows out_stride wide (a head's vector holds more than the map reads or writes). Float32 sums, each output summed over k
// in order by one thread: a function of the row alone.
#define HL_TILE 64          // rows and columns of a workgroup's tile
#define HL_K 16             // k values staged at a time
template <typename TI, typename TW, typename TO>
__global__ __launch_bounds__(256) void head_linear_kernel(const TI* __restrict__ in, int in_stride, const TW* __restrict__ w,
                                                         const float* __restrict__ gate, int gate_stride, TO* __restrict__ out,
                                                         int rows, int heads, int N, int K, int in_head, int out_head, int out_stride) {
    __shared__ float a_tile[HL_K][HL_TILE + 1], w_tile[HL_K][HL_TILE + 1];
    const int head = blockIdx.z;
    const int row0 = blockIdx.x * HL_TILE, col0 = blockIdx.y * HL_TILE;
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const TW* w_head = w + (size_t)head * N * K;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += HL_K) {
        // 64 x 16 of each operand: four values a thread
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int item = threadIdx.x + 256 * u;
            const int line = item / HL_K, k = item % HL_K;
            const bool k_in = k0 + k < K;
            a_tile[k][line] = (k_in && row0 + line < rows) ? load_as_float(in, (size_t)(row0 + line) * in_stride + (size_t)head * in_head + k0 + k) : 0.0f;
            w_tile[k][line] = (k_in && col0 + line < N) ? load_as_float(w_head, (size_t)(col0 + line) * K + k0 + k) : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < HL_K; ++k) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                av[i] = a_tile[k][ty + 16 * i];
                wv[i] = w_tile[k][tx + 16 * i];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = row0 + ty + 16 * i;
        if (row >= rows) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = col0 + tx + 16 * j;
            if (col >= N) continue;
            float value = acc[i][j];
            if (gate) {
                const float z = gate[(size_t)row * gate_stride + (size_t)head * N + col];
                value *= 1.0f / (1.0f + expf(-z));
            }
            store_from_float(out, (size_t)row * out_stride + (size_t)head * out_head + col, value);
        }
    }
}

// Few rows of float32 inputs against bfloat16 weights (a decode step's gates of a recurrence, which stay float32): a wave
// per output, its lanes along k, every row's sum through the wave; the weights are read once, in runs along k. Float32
// products and sums; a row's sum does not depend on the rows beside it.
#define HL_FEW_ROWS 16
// VEC: K, the rows' stride and the heads' offsets are multiples of 4 and the pointers 16-byte aligned: a lane takes four
// neighbouring k at a time, the weights' as one 8-byte load and each row's as one of 16 bytes, all asked for together.
template <bool VEC>
__global__ __launch_bounds__(256) void head_linear_few_rows_kernel(const float* __restrict__ in, int in_stride, const uint16_t* __restrict__ w,
                                                                  float* __restrict__ out, int rows, int heads, int N, int K, int in_head,
                                                                  int out_head, int out_stride) {
    const int head = blockIdx.y;
    const int n = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (n >= N) return;
    const uint16_t* w_row = w + ((size_t)head * N + n) * K;
    const float* from = in + (size_t)head * in_head;
    float acc[HL_FEW_ROWS];
#pragma unroll
    for (int r = 0; r < HL_FEW_ROWS; ++r) acc[r] = 0.0f;
    if (VEC) {
        typedef __attribute__((ext_vector_type(4))) float f32x4_t;
        typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;
        for (int k = lane * 4; k < K; k += 256) {
            const u32x2_t bits = *reinterpret_cast<const u32x2_t*>(w_row + k);
            f32x4_t x[HL_FEW_ROWS];
#pragma unroll
            for (int r = 0; r < HL_FEW_ROWS; ++r) x[r] = *reinterpret_cast<const f32x4_t*>(from + (size_t)(r < rows ? r : rows - 1) * in_stride + k);
            const float w0 = __uint_as_float(bits[0] << 16), w1 = __uint_as_float(bits[0] & 0xffff0000u);
            const float w2 = __uint_as_float(bits[1] << 16), w3 = __uint_as_float(bits[1] & 0xffff0000u);
#pragma unroll
            for (int r = 0; r < HL_FEW_ROWS; ++r) acc[r] = fmaf(x[r][3], w3, fmaf(x[r][2], w2, fmaf(x[r][1], w1, fmaf(x[r][0], w0, acc[r]))));
        }
    } else {
        for (int k = lane; k < K; k += 64) {
            const float wv = __uint_as_float((uint32_t)w_row[k] << 16);
#pragma unroll
            for (int r = 0; r < HL_FEW_ROWS; ++r)
                if (r < rows) acc[r] = fmaf(from[(size_t)r * in_stride + k], wv, acc[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < HL_FEW_ROWS; ++r) {
        if (r >= rows) break;
        const float sum = wave_sum(acc[r]);
        if (lane == 0) out[(size_t)r * out_stride + (size_t)head * out_head + n] = sum;
    }
}

// The same on the matrix cores, bfloat16 in, float32 sums, bfloat16 out. A wave forms 16 rows by 16 NT outputs of
// one head: per 32 values of k one operand of the rows and NT of the weights, each lane's eight values
// one 16-byte load straight from memory (K and the rows' stride multiples of 8), no LDS: the weights of a head are
// few and stay in the caches for the waves that share them. The product is taken transposed (weights as
// the first operand), so that a lane ends with four neighbouring outputs of one row. WIDE: the workgroup's
// four waves take four runs of outputs of the same 16 rows (a decode step's few rows); else four runs of
// rows for the same outputs. Each output's sum runs over k in the same order whatever the rows beside it.
typedef __attribute__((ext_vector_type(8))) __bf16 hl_bf16x8;
typedef __attribute__((ext_vector_type(4))) float hl_f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t hl_u32x4;
template <int NT, bool WIDE>
__global__ __launch_bounds__(256) void head_linear_mfma_kernel(const uint16_t* __restrict__ in, int in_stride, const uint16_t* __restrict__ w,
                                                              const float* __restrict__ gate, int gate_stride, uint16_t* __restrict__ out,
                                                              int rows, int heads, int N, int K, int in_head, int out_head, int out_stride) {
    const int head = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, i16 = lane & 15, g = lane >> 4;
    const int row0 = WIDE ? blockIdx.x * 16 : (blockIdx.x * 4 + wave) * 16;
    const int col0 = WIDE ? (blockIdx.y * 4 + wave) * 16 * NT : blockIdx.y * 16 * NT;
    if (row0 >= rows || col0 >= N) return;
    const int my_row = row0 + i16 < rows ? row0 + i16 : rows - 1;           // rows past the end compute along and store nothing
    const uint16_t* a_from = in + (size_t)my_row * in_stride + (size_t)head * in_head + g * 8;
    const uint16_t* w_from[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int n = col0 + t * 16 + i16 < N ? col0 + t * 16 + i16 : N - 1;
        w_from[t] = w + ((size_t)head * N + n) * K + g * 8;
    }
    hl_f32x4 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = hl_f32x4{0.f, 0.f, 0.f, 0.f};
    const hl_u32x4 zero = {0u, 0u, 0u, 0u};
    for (int k0 = 0; k0 < K; k0 += 32) {
        const bool k_in = k0 + g * 8 < K;
        const hl_u32x4 a_bits = k_in ? *reinterpret_cast<const hl_u32x4*>(a_from + k0) : zero;
        hl_u32x4 w_bits[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) w_bits[t] = k_in ? *reinterpret_cast<const hl_u32x4*>(w_from[t] + k0) : zero;
#pragma unroll
        for (int t = 0; t < NT; ++t)
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(hl_bf16x8, w_bits[t]), __builtin_bit_cast(hl_bf16x8, a_bits), acc[t], 0, 0, 0);
    }
    fw_mfma_drain();        // the last products have left the pipe before a branch leads to code that reads them
    if (row0 + i16 >= rows) return;
    const int row = row0 + i16;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int n0 = col0 + t * 16 + g * 4;           // this lane: outputs n0 .. n0 + 3 of its row
        float value[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            value[r] = acc[t][r];
            if (gate && n0 + r < N) value[r] *= 1.0f / (1.0f + expf(-gate[(size_t)row * gate_stride + (size_t)head * N + n0 + r]));
        }
        uint16_t* dest = out + (size_t)row * out_stride + (size_t)head * out_head + n0;
        if (n0 + 3 < N && N % 4 == 0) {
            typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
            *reinterpret_cast<u32x2*>(dest) = u32x2{(uint32_t)float_to_bf16_bits(value[0]) | ((uint32_t)float_to_bf16_bits(value[1]) << 16),
                                                    (uint32_t)float_to_bf16_bits(value[2]) | ((uint32_t)float_to_bf16_bits(value[3]) << 16)};
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n0 + r < N) dest[r] = float_to_bf16_bits(value[r]);
        }
    }
}

extern "C" int fw_head_linear(const void* in, int in_dtype, int in_stride, const void* w, int w_dtype, const float* gate,
                              int gate_stride, void* out, int out_dtype, int rows, int heads, int N, int K, int in_head, int out_head,
                              int out_stride, void* stream) {
    FW_REQUIRE(rows >= 0 && heads > 0 && heads <= 65535 && N > 0 && K > 0, "head_linear: bad sizes rows=%d heads=%d N=%d K=%d", rows, heads, N, K);
    if (in_head <= 0) in_head = K;
    if (out_head <= 0) out_head = N;
    if (out_stride <= 0) out_stride = heads * out_head;
    FW_REQUIRE(in_head >= K && in_stride >= (heads - 1) * in_head + K, "head_linear: rows %d wide do not hold %d heads %d apart of %d", in_stride, heads, in_head, K);
    FW_REQUIRE(out_head >= N && out_stride >= (heads - 1) * out_head + N, "head_linear: rows %d wide do not take %d heads %d apart of %d", out_stride, heads, out_head, N);
    FW_REQUIRE(gate == nullptr || (out_head == N && out_stride == heads * N), "head_linear: a gate goes with outputs side by side");
    FW_REQUIRE(gate == nullptr || gate_stride >= heads * N, "head_linear: the gates' rows (%d wide) do not hold %d x %d", gate_stride, heads, N);
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (in_dtype == FW_BF16 && w_dtype == FW_BF16 && out_dtype == FW_BF16 && K % 8 == 0 && in_stride % 8 == 0 && in_head % 8 == 0 &&
        (uintptr_t)in % 16 == 0 && (uintptr_t)w % 16 == 0 && (uintptr_t)out % 8 == 0 && out_head % 4 == 0 && out_stride % 4 == 0) {
        // few rows: a wave per 16 outputs, so that a small product still spreads over the chip; else 64 outputs a wave
        if (rows <= 16) {
            dim3 wide(1, (N + 63) / 64, heads);
            FW_REQUIRE(wide.y <= 65535, "head_linear: too many columns (%d)", N);
            head_linear_mfma_kernel<1, true><<<wide, 256, 0, s>>>((const uint16_t*)in, in_stride, (const uint16_t*)w, gate, gate_stride,
                                                                  (uint16_t*)out, rows, heads, N, K, in_head, out_head, out_stride);
        } else {
            dim3 tall((rows + 63) / 64, (N + 63) / 64, heads);
            FW_REQUIRE(tall.y <= 65535, "head_linear: too many columns (%d)", N);
            head_linear_mfma_kernel<4, false><<<tall, 256, 0, s>>>((const uint16_t*)in, in_stride, (const uint16_t*)w, gate, gate_stride,
                                                                   (uint16_t*)out, rows, heads, N, K, in_head, out_head, out_stride);
        }
        FW_LAUNCH_CHECK("head_linear");
        return 0;
    }
    if (rows <= HL_FEW_ROWS && in_dtype == FW_F32 && w_dtype == FW_BF16 && out_dtype == FW_F32 && gate == nullptr) {
        const bool vec = K % 4 == 0 && in_stride % 4 == 0 && in_head % 4 == 0 && (uintptr_t)in % 16 == 0 && (uintptr_t)w % 8 == 0;
        if (vec)
            head_linear_few_rows_kernel<true><<<dim3((N + 3) / 4, heads), 256, 0, s>>>((const float*)in, in_stride, (const uint16_t*)w, (float*)out,
                                                                                       rows, heads, N, K, in_head, out_head, out_stride);
        else
            head_linear_few_rows_kernel<false><<<dim3((N + 3) / 4, heads), 256, 0, s>>>((const float*)in, in_stride, (const uint16_t*)w, (float*)out,
                                                                                        rows, heads, N, K, in_head, out_head, out_stride);
        FW_LAUNCH_CHECK("head_linear");
        return 0;
    }
    dim3 grid((rows + HL_TILE - 1) / HL_TILE, (N + HL_TILE - 1) / HL_TILE, heads);
    FW_REQUIRE(grid.y <= 65535, "head_linear: too many columns (%d)", N);
#define FW_HL_LAUNCH(TI, TW, TO)                                                                                          \
    head_linear_kernel<TI, TW, TO><<<grid, 256, 0, s>>>((const TI*)in, in_stride, (const TW*)w, gate, gate_stride, \
                                                        (TO*)out, rows, heads, N, K, in_head, out_head, out_stride)
    if (in_dtype == FW_F32 && w_dtype == FW_F32 && out_dtype == FW_F32) FW_HL_LAUNCH(float, float, float);
    else if (in_dtype == FW_BF16 && w_dtype == FW_BF16 && out_dtype == FW_BF16) FW_HL_LAUNCH(bf16_t, bf16_t, bf16_t);
    else if (in_dtype == FW_BF16 && w_dtype == FW_BF16 && out_dtype == FW_F32) FW_HL_LAUNCH(bf16_t, bf16_t, float);
    else if (in_dtype == FW_F32 && w_dtype == FW_BF16 && out_dtype == FW_BF16) FW_HL_LAUNCH(float, bf16_t, bf16_t);
    else if (in_dtype == FW_F32 && w_dtype == FW_BF16 && out_dtype == FW_F32) FW_HL_LAUNCH(float, bf16_t, float);
    else FW_REQUIRE(false, "head_linear: unsupported dtypes in=%d w=%d out=%d", in_dtype, w_dtype, out_dtype);
#undef FW_HL_LAUNCH
    FW_LAUNCH_CHECK("head_linear");
    return 0;
}

// ---- a rotated part of every head's vector -------------------------------------------------------------------
// in [rows][in_stride]: head h's vector begins at h * in_head and its channels col0 .. col0 + rot - 1 are turned
// (neighbouring channels (2i, 2i + 1) of the first `turn` by the row's angles, tables [rows][turn / 2], float32; the rest pass) and stored at
// out[r][h * out_head + out_col0 ..] in rows out_stride wide. A thread per (row, head, pair).
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void rotate_place_kernel(const TI* __restrict__ in, int in_stride, int in_head, int col0,
                                                          const float* __restrict__ cos_table, const float* __restrict__ sin_table,
                                                          TO* __restrict__ out, int out_stride, int out_head, int out_col0, int heads,
                                                          int rot, int turn) {
    const int row = blockIdx.x, half = rot / 2, turned = turn / 2;
    for (int item = threadIdx.x; item < heads * half; item += blockDim.x) {
        const int head = item / half, pair = item % half;
        const TI* source = in + (size_t)row * in_stride + (size_t)head * in_head + col0;
        const float u = load_as_float(source, 2 * pair), v = load_as_float(source, 2 * pair + 1);
        // a pair past the turned channels passes as it is (an angle of zero)
        const float c = pair < turned ? cos_table[(size_t)row * turned + pair] : 1.0f;
        const float sn = pair < turned ? sin_table[(size_t)row * turned + pair] : 0.0f;
        TO* dest = out + (size_t)row * out_stride + (size_t)head * out_head + out_col0;
        store_from_float(dest, 2 * pair, fmaf(u, c, -(v * sn)));
        store_from_float(dest, 2 * pair + 1, fmaf(v, c, u * sn));
    }
}

extern "C" int fw_rotate_place(const void* in, int in_dtype, int in_stride, int in_head, int col0, const float* cos_table,
                               const float* sin_table, void* out, int out_dtype, int out_stride, int out_head, int out_col0, int rows,
                               int heads, int rot, int turn, void* stream) {
    FW_REQUIRE(turn >= 0 && turn <= rot && turn % 2 == 0, "rotate_place: %d turned channels of %d", turn, rot);
    FW_REQUIRE(rows >= 0 && heads > 0 && rot > 0 && rot % 2 == 0, "rotate_place: bad sizes rows=%d heads=%d rot=%d", rows, heads, rot);
    FW_REQUIRE(col0 >= 0 && col0 + rot <= in_head && in_stride >= (heads - 1) * in_head + col0 + rot,
               "rotate_place: rows %d wide do not hold %d heads %d apart with channels %d..%d", in_stride, heads, in_head, col0, col0 + rot);
    FW_REQUIRE(out_col0 >= 0 && out_col0 + rot <= out_head && out_stride >= (heads - 1) * out_head + out_col0 + rot,
               "rotate_place: rows %d wide do not take %d heads %d apart with channels %d..%d", out_stride, heads, out_head, out_col0, out_col0 + rot);
    FW_REQUIRE(turn == 0 || (cos_table && sin_table), "rotate_place: the rotation tables are missing");
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
#define FW_RP_LAUNCH(TI, TO)                                                                                                      \
    rotate_place_kernel<TI, TO><<<rows, 256, 0, s>>>((const TI*)in, in_stride, in_head, col0, cos_table, sin_table, (TO*)out, out_stride, \
                                                     out_head, out_col0, heads, rot, turn)
    if (in_dtype == FW_F32 && out_dtype == FW_F32) FW_RP_LAUNCH(float, float);
    else if (in_dtype == FW_BF16 && out_dtype == FW_BF16) FW_RP_LAUNCH(bf16_t, bf16_t);
    else if (in_dtype == FW_F32 && out_dtype == FW_BF16) FW_RP_LAUNCH(float, bf16_t);
    else FW_REQUIRE(false, "rotate_place: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
#undef FW_RP_LAUNCH
    FW_LAUNCH_CHECK("rotate_place");
    return 0;
}
