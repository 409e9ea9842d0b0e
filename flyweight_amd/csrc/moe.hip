// A mixture of small feed-forward units chosen per token.
//
//   fw_moe_route      the `top` largest router logits of every row (ties: the lowest id) and the softmax over them
//   fw_moe_arrange    the (row, choice) pairs sorted by expert, stably: where each expert's pairs begin, which
//                     row a place holds, which place a pair got
//   fw_grouped_gemm   out[place] = a[row of place] . W[expert of place]^T for all places, a tile of places
//                     belonging to one expert; storing, or the gated unit silu(gate) * up
//   fw_moe_combine    x[row] += sum over the row's choices, in the order of the choices, of weight * y[place]
//
// Everything that decides (logits, choice, weights) and every sum is float32; the order of every sum
// depends on the row alone, never on what else is in the step.
#include "fw_common.h"
#include "fw_kernels.h"

// ---- routing ---------------------------------------------------------------------------------------
// A wave per row. The logits (float32 [rows][experts], bias added here) stay in registers, up to
// MOE_MAX_EXPERTS / 64 a lane; `top` rounds of a wave-wide best-of, each taking the winner out.
#define MOE_MAX_EXPERTS 1024
#define MOE_MAX_TOP 64
__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ logits, const float* __restrict__ bias,
                                                      int32_t* __restrict__ chosen, float* __restrict__ weight, int experts, int top) {
    const int row = blockIdx.x, lane = threadIdx.x;
    float z[MOE_MAX_EXPERTS / 64];
#pragma unroll
    for (int i = 0; i < MOE_MAX_EXPERTS / 64; ++i) {
        const int e = lane + 64 * i;
        z[i] = e < experts ? logits[(size_t)row * experts + e] + (bias ? bias[e] : 0.0f) : -INFINITY;
    }
    float first = 0.0f, total = 0.0f, mine = 0.0f;      // lane j keeps the j-th choice's exponential
    for (int round = 0; round < top; ++round) {
        float best = -INFINITY;
        int best_id = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < MOE_MAX_EXPERTS / 64; ++i) {
            const int e = lane + 64 * i;
            if (e < experts && (z[i] > best || (z[i] == best && e < best_id))) {
                best = z[i];
                best_id = e;
            }
        }
#pragma unroll
        for (int offset = 32; offset > 0; offset >>= 1) {
            const float other = __shfl_xor(best, offset, 64);
            const int other_id = __shfl_xor(best_id, offset, 64);
            if (other > best || (other == best && other_id < best_id)) {
                best = other;
                best_id = other_id;
            }
        }
#pragma unroll
        for (int i = 0; i < MOE_MAX_EXPERTS / 64; ++i)
            if (lane + 64 * i == best_id) z[i] = -INFINITY;
        if (round == 0) first = best;                   // the largest: the softmax's shift
        const float e = expf(best - first);
        total += e;
        if (lane == round) {
            mine = e;
            chosen[(size_t)row * top + round] = best_id;
        }
    }
    if (lane < top) weight[(size_t)row * top + lane] = mine / total;
}

extern "C" int fw_moe_route(const float* logits, const float* bias, int32_t* chosen, float* weight, int rows, int experts, int top,
                            void* stream) {
    FW_REQUIRE(rows >= 0 && experts >= 1 && experts <= MOE_MAX_EXPERTS, "moe_route: %d experts (1..%d)", experts, MOE_MAX_EXPERTS);
    FW_REQUIRE(top >= 1 && top <= experts && top <= MOE_MAX_TOP, "moe_route: %d of %d experts a token (at most %d)", top, experts, MOE_MAX_TOP);
    if (rows == 0) return 0;
    moe_route_kernel<<<rows, 64, 0, (hipStream_t)stream>>>(logits, bias, chosen, weight, experts, top);
    FW_LAUNCH_CHECK("moe_route");
    return 0;
}

// ---- sorting the pairs by expert ------------------------------------------------------------------------
// One workgroup. Pass 1 counts the pairs of every expert (LDS counters), a scan gives where each expert
// begins, pass 2 hands out places: a thread takes a contiguous run of pairs, in order, and the runs of one
// expert follow each other in the order of the threads, so that an expert's places hold its pairs in the
// order (row, choice). expert_begin [experts + 1]; place_row [pairs]; pair_place [pairs].
#define MOE_ARRANGE_THREADS 1024
__global__ __launch_bounds__(MOE_ARRANGE_THREADS) void moe_arrange_kernel(const int32_t* __restrict__ chosen, int32_t* __restrict__ expert_begin,
                                                                          int32_t* __restrict__ place_row, int32_t* __restrict__ pair_place,
                                                                          int pairs, int experts, int top) {
    extern __shared__ int32_t counts[];         // [experts + 1] begins, then [threads-in-use][experts] is too much: runs are walked twice instead
    const int tid = threadIdx.x;
    for (int e = tid; e <= experts; e += MOE_ARRANGE_THREADS) counts[e] = 0;
    __syncthreads();
    for (int i = tid; i < pairs; i += MOE_ARRANGE_THREADS) atomicAdd(&counts[chosen[i]], 1);
    __syncthreads();
    if (tid == 0) {
        int running = 0;
        for (int e = 0; e < experts; ++e) {
            const int n = counts[e];
            counts[e] = running;
            running += n;
        }
        counts[experts] = running;
    }
    __syncthreads();
    for (int e = tid; e <= experts; e += MOE_ARRANGE_THREADS) expert_begin[e] = counts[e];
    // Places in order: a wave per expert at a time walks all pairs in runs of 64 and numbers those of its
    // expert by a prefix count over the lanes (ballot), so the order is that of the pairs.
    const int lane = tid & 63, wave = tid >> 6, waves = MOE_ARRANGE_THREADS / 64;
    for (int e = wave; e < experts; e += waves) {
        int next = counts[e];
        const int end = e + 1 <= experts ? counts[e + 1] : pairs;
        if (next == end) continue;
        for (int i0 = 0; i0 < pairs; i0 += 64) {
            const int i = i0 + lane;
            const bool is_mine = i < pairs && chosen[i] == e;
            const unsigned long long votes = __ballot(is_mine);
            if (is_mine) {
                const int place = next + __popcll(votes & ((1ull << lane) - 1ull));
                place_row[place] = i / top;
                pair_place[i] = place;
            }
            next += __popcll(votes);
        }
    }
}

extern "C" int fw_moe_arrange(const int32_t* chosen, int32_t* expert_begin, int32_t* place_row, int32_t* pair_place, int rows, int experts,
                              int top, void* stream) {
    FW_REQUIRE(rows >= 0 && experts >= 1 && experts <= MOE_MAX_EXPERTS && top >= 1, "moe_arrange: bad sizes rows=%d experts=%d top=%d", rows, experts, top);
    FW_REQUIRE((long long)rows * top < (1ll << 30), "moe_arrange: too many pairs");
    moe_arrange_kernel<<<1, MOE_ARRANGE_THREADS, (experts + 1) * sizeof(int32_t), (hipStream_t)stream>>>(chosen, expert_begin, place_row, pair_place,
                                                                                                        rows * top, experts, top);
    FW_LAUNCH_CHECK("moe_arrange");
    return 0;
}

// ---- the grouped product, plain form ------------------------------------------------------------------
// Tiles of GG_ROWS places x GG_COLS features; a tile's places belong to one expert. blockIdx.x numbers
// the row tiles of all experts one after the other (an expert with n places has ceil(n / GG_ROWS)); the
// grid holds as many as there can be at most, a workgroup beyond the last tile leaves at once. A thread
// computes 2 x 4 outputs; each output is summed over k in order by one thread. a: [*, K] rows, taken at
// place_row[place] (or at the place itself when place_row is null); w: [experts][N (x 2)][K].
#define GG_ROWS 32
#define GG_COLS 64
#define GG_K 16
template <typename TA, typename TW, typename TO, bool GATED>
__global__ __launch_bounds__(256) void grouped_gemm_kernel(const TA* __restrict__ a, const int32_t* __restrict__ place_row,
                                                          const TW* __restrict__ w, const int32_t* __restrict__ expert_begin,
                                                          TO* __restrict__ out, int experts, int N, int K) {
    __shared__ float as[GG_K][GG_ROWS + 1];
    __shared__ float ws[GATED ? 2 : 1][GG_K][GG_COLS + 1];
    __shared__ int tile_expert, tile_first, tile_end;
    if (threadIdx.x == 0) {
        int tile = blockIdx.x, found = -1, first = 0, end = 0;
        for (int e = 0; e < experts; ++e) {
            const int begin = expert_begin[e], stop = expert_begin[e + 1];
            const int tiles = (stop - begin + GG_ROWS - 1) / GG_ROWS;
            if (tile < tiles) {
                found = e;
                first = begin + tile * GG_ROWS;
                end = stop;
                break;
            }
            tile -= tiles;
        }
        tile_expert = found;
        tile_first = first;
        tile_end = end;
    }
    __syncthreads();
    const int expert = tile_expert;
    if (expert < 0) return;
    const int first = tile_first, count = tile_end - first < GG_ROWS ? tile_end - first : GG_ROWS;
    const int col0 = blockIdx.y * GG_COLS;
    const int tid = threadIdx.x;
    const int tr = tid / 16, tc = tid % 16;             // rows 2 tr, 2 tr + 1; columns tc, tc + 16, tc + 32, tc + 48
    const size_t rows_of_w = GATED ? 2 * (size_t)N : (size_t)N;
    const TW* we = w + (size_t)expert * rows_of_w * K;
    float acc[GATED ? 2 : 1][2][4] = {};
    // what this thread copies of every slab: a's element (row la_r, k la_k x 2), w's (column lw_c, k lw_k x 4)
    const int la_r = tid / 8, la_k = (tid % 8) * 2;
    const int lw_c = tid / 4, lw_k = (tid % 4) * 4;
    const int a_row = la_r < count ? (place_row ? place_row[first + la_r] : first + la_r) : -1;
    for (int k0 = 0; k0 < K; k0 += GG_K) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int kk = k0 + la_k + j;
            as[la_k + j][la_r] = (a_row >= 0 && kk < K) ? load_as_float(a, (size_t)a_row * K + kk) : 0.0f;
        }
#pragma unroll
        for (int half = 0; half < (GATED ? 2 : 1); ++half)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int kk = k0 + lw_k + j, col = col0 + lw_c;
                ws[half][lw_k + j][lw_c] = (col < N && kk < K) ? load_as_float(we, ((size_t)half * N + col) * K + kk) : 0.0f;
            }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GG_K; ++kk) {
            const float a0 = as[kk][2 * tr], a1 = as[kk][2 * tr + 1];
#pragma unroll
            for (int half = 0; half < (GATED ? 2 : 1); ++half)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float b = ws[half][kk][tc + 16 * j];
                    acc[half][0][j] = fmaf(a0, b, acc[half][0][j]);
                    acc[half][1][j] = fmaf(a1, b, acc[half][1][j]);
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = 2 * tr + i;
        if (r >= count) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = col0 + tc + 16 * j;
            if (col >= N) continue;
            float value = acc[0][i][j];
            if (GATED) {
                const float g = acc[0][i][j];
                value = g / (1.0f + expf(-g)) * acc[1][i][j];
            }
            store_from_float(out, (size_t)(first + r) * N + col, value);
        }
    }
}

extern "C" int fw_grouped_gemm(const void* a, int a_dtype, const int32_t* place_row, const void* w, int w_dtype,
                               const int32_t* expert_begin, void* out, int out_dtype, int gated, int places, int experts, int N, int K,
                               void* stream) {
    FW_REQUIRE(places >= 0 && experts >= 1 && N > 0 && K > 0, "grouped_gemm: bad sizes places=%d experts=%d N=%d K=%d", places, experts, N, K);
    if (places == 0) return 0;
    const long long tiles = (long long)places / GG_ROWS + experts;      // at most: every expert may end in a tile that is not full
    FW_REQUIRE(tiles < (1ll << 31) && (N + GG_COLS - 1) / GG_COLS <= 65535, "grouped_gemm: grid too large");
    dim3 grid((unsigned)tiles, (N + GG_COLS - 1) / GG_COLS);
    hipStream_t s = (hipStream_t)stream;
#define FW_GG_LAUNCH(TA, TW, TO)                                                                                                   \
    {                                                                                                                              \
        if (gated) grouped_gemm_kernel<TA, TW, TO, true><<<grid, 256, 0, s>>>((const TA*)a, place_row, (const TW*)w, expert_begin, \
                                                                              (TO*)out, experts, N, K);                           \
        else grouped_gemm_kernel<TA, TW, TO, false><<<grid, 256, 0, s>>>((const TA*)a, place_row, (const TW*)w, expert_begin,      \
                                                                         (TO*)out, experts, N, K);                                \
    }
    if (a_dtype == FW_F32 && w_dtype == FW_F32 && out_dtype == FW_F32) FW_GG_LAUNCH(float, float, float)
    else if (a_dtype == FW_BF16 && w_dtype == FW_BF16 && out_dtype == FW_BF16) FW_GG_LAUNCH(bf16_t, bf16_t, bf16_t)
    else if (a_dtype == FW_BF16 && w_dtype == FW_BF16 && out_dtype == FW_F32) FW_GG_LAUNCH(bf16_t, bf16_t, float)
    else FW_REQUIRE(false, "grouped_gemm: unsupported dtypes a=%d w=%d out=%d", a_dtype, w_dtype, out_dtype);
#undef FW_GG_LAUNCH
    FW_LAUNCH_CHECK("grouped_gemm");
    return 0;
}

// ---- back to the rows ---------------------------------------------------------------------------------
// x[row] += sum_j weight[row][j] * y[pair_place[row][j]], the choices in their order; float32.
__global__ void moe_combine_kernel(float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ weight,
                                   const int32_t* __restrict__ pair_place, int top, int hidden) {
    const int row = blockIdx.y;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < hidden; i += gridDim.x * blockDim.x) {
        float sum = 0.0f;
        for (int j = 0; j < top; ++j)
            sum = fmaf(weight[(size_t)row * top + j], y[(size_t)pair_place[(size_t)row * top + j] * hidden + i], sum);
        x[(size_t)row * hidden + i] += sum;
    }
}

extern "C" int fw_moe_combine(float* x, const float* y, const float* weight, const int32_t* pair_place, int rows, int top, int hidden,
                              void* stream) {
    FW_REQUIRE(rows >= 0 && rows <= 65535 && top >= 1 && hidden > 0, "moe_combine: bad sizes rows=%d top=%d hidden=%d", rows, top, hidden);
    if (rows == 0) return 0;
    dim3 grid(fw_ceil_div(hidden, 256) > 64 ? 64 : fw_ceil_div(hidden, 256), rows);
    moe_combine_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(x, y, weight, pair_place, top, hidden);
    FW_LAUNCH_CHECK("moe_combine");
    return 0;
}
