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
// groups > 1: the experts form that many equal groups of neighbours, a group's score is its best expert's, and only
// experts of the `keep` best groups (ties: the lowest group) can be chosen. score_all: the weights are the softmax
// over ALL experts at the chosen ones, divided by their sum + 1e-20 (else the softmax over the chosen alone).
__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ logits, const float* __restrict__ bias,
                                                      int32_t* __restrict__ chosen, float* __restrict__ weight, int experts, int top,
                                                      int groups, int keep, int score_all) {
    const int row = blockIdx.x, lane = threadIdx.x;
    float z[MOE_MAX_EXPERTS / 64];
#pragma unroll
    for (int i = 0; i < MOE_MAX_EXPERTS / 64; ++i) {
        const int e = lane + 64 * i;
        z[i] = e < experts ? logits[(size_t)row * experts + e] + (bias ? bias[e] : 0.0f) : -INFINITY;
    }
    float all_max = 0.0f, all_sum = 1.0f;
    if (score_all) {    // the softmax's maximum and sum over every expert, before any is shut out
        float m = -INFINITY;
#pragma unroll
        for (int i = 0; i < MOE_MAX_EXPERTS / 64; ++i) m = fmaxf(m, z[i]);
        all_max = wave_max(m);
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < MOE_MAX_EXPERTS / 64; ++i)
            if (lane + 64 * i < experts) sum += expf(z[i] - all_max);
        all_sum = wave_sum(sum);
    }
    if (groups > 1 && keep < groups) {
        // lane g holds the best logit of group g (the softmax is monotonic: the best score is the best logit's)
        const int per_group = experts / groups;
        float group_best = -INFINITY;
        for (int g = 0; g < groups; ++g) {
            float m = -INFINITY;
#pragma unroll
            for (int i = 0; i < MOE_MAX_EXPERTS / 64; ++i) {
                const int e = lane + 64 * i;
                if (e < experts && e / per_group == g) m = fmaxf(m, z[i]);
            }
            m = wave_max(m);
            if (lane == g) group_best = m;
        }
        unsigned long long kept = 0ull;
        for (int round = 0; round < keep; ++round) {
            // a group already taken is no longer offered
            const bool offered = lane < groups && !((kept >> lane) & 1ull);
            float best = offered ? group_best : -INFINITY;
            int best_id = offered ? lane : 0x7fffffff;
#pragma unroll
            for (int offset = 32; offset > 0; offset >>= 1) {
                const float other = __shfl_xor(best, offset, 64);
                const int other_id = __shfl_xor(best_id, offset, 64);
                if (other_id < 0x7fffffff && (best_id == 0x7fffffff || other > best || (other == best && other_id < best_id))) {
                    best = other;
                    best_id = other_id;
                }
            }
            kept |= 1ull << best_id;        // every lane holds the same winner
        }
#pragma unroll
        for (int i = 0; i < MOE_MAX_EXPERTS / 64; ++i) {
            const int e = lane + 64 * i;
            if (e < experts && !((kept >> (e / per_group)) & 1ull)) z[i] = -INFINITY;
        }
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
        const float e = score_all ? expf(best - all_max) / all_sum : expf(best - first);
        total += e;
        if (lane == round) {
            mine = e;
            chosen[(size_t)row * top + round] = best_id;
        }
    }
    if (lane < top) weight[(size_t)row * top + lane] = mine / (score_all ? total + 1e-20f : total);
}

extern "C" int fw_moe_route(const float* logits, const float* bias, int32_t* chosen, float* weight, int rows, int experts, int top,
                            int groups, int keep, int score_all, void* stream) {
    if (groups <= 0) groups = 1;
    if (keep <= 0) keep = groups;
    FW_REQUIRE(groups <= 64 && experts % groups == 0 && keep <= groups, "moe_route: %d experts in %d groups (at most 64, equal ones) of which %d are kept",
               experts, groups, keep);
    FW_REQUIRE(top <= keep * (experts / groups), "moe_route: %d experts a token cannot come from %d groups of %d", top, keep, experts / groups);
    FW_REQUIRE(rows >= 0 && experts >= 1 && experts <= MOE_MAX_EXPERTS, "moe_route: %d experts (1..%d)", experts, MOE_MAX_EXPERTS);
    FW_REQUIRE(top >= 1 && top <= experts && top <= MOE_MAX_TOP, "moe_route: %d of %d experts a token (at most %d)", top, experts, MOE_MAX_TOP);
    if (rows == 0) return 0;
    moe_route_kernel<<<rows, 64, 0, (hipStream_t)stream>>>(logits, bias, chosen, weight, experts, top, groups, keep, score_all);
    FW_LAUNCH_CHECK("moe_route");
    return 0;
}

// ---- sorting the pairs by expert ------------------------------------------------------------------------
// One workgroup of 16 waves; the pairs are cut into 16 runs, one a wave, in order. Pass 1: every wave counts
// its run's pairs per expert (LDS counters [wave][expert]). A thread per expert then turns the counts into
// where the expert begins (a scan over the experts by one thread) and where each wave's pairs of it begin.
// Pass 2: every wave walks its run 64 pairs at a time; the lanes that chose the same expert number themselves
// by a prefix count (ballot), one expert after the other, behind the wave's running place for that expert.
// So an expert's places hold its pairs in the order (row, choice), whatever the timing.
// expert_begin [experts + 1]; place_row [pairs]; pair_place [pairs].
#define MOE_ARRANGE_THREADS 1024
#define MOE_ARRANGE_WAVES (MOE_ARRANGE_THREADS / 64)
__global__ __launch_bounds__(MOE_ARRANGE_THREADS) void moe_arrange_kernel(const int32_t* __restrict__ chosen, int32_t* __restrict__ expert_begin,
                                                                          int32_t* __restrict__ place_row, int32_t* __restrict__ pair_place,
                                                                          int pairs, int experts, int top) {
    extern __shared__ int32_t counts[];         // [waves][experts] counts, then running places; behind them [experts + 1] begins
    int32_t* begins = counts + MOE_ARRANGE_WAVES * experts;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int run = ((pairs + MOE_ARRANGE_WAVES - 1) / MOE_ARRANGE_WAVES + 63) / 64 * 64;    // pairs of a wave, whole rounds of 64
    const int run0 = wave * run, run_end = run0 + run < pairs ? run0 + run : pairs;
    for (int i = tid; i < MOE_ARRANGE_WAVES * experts; i += MOE_ARRANGE_THREADS) counts[i] = 0;
    __syncthreads();
    for (int i = run0 + lane; i < run_end; i += 64) atomicAdd(&counts[wave * experts + chosen[i]], 1);
    __syncthreads();
    for (int e = tid; e < experts; e += MOE_ARRANGE_THREADS) {
        int total = 0;
        for (int w = 0; w < MOE_ARRANGE_WAVES; ++w) total += counts[w * experts + e];
        begins[e] = total;
    }
    __syncthreads();
    if (tid == 0) {
        int running = 0;
        for (int e = 0; e < experts; ++e) {
            const int n = begins[e];
            begins[e] = running;
            running += n;
        }
        begins[experts] = running;
    }
    __syncthreads();
    for (int e = tid; e <= experts; e += MOE_ARRANGE_THREADS) expert_begin[e] = begins[e];
    for (int e = tid; e < experts; e += MOE_ARRANGE_THREADS) {
        int running = begins[e];
        for (int w = 0; w < MOE_ARRANGE_WAVES; ++w) {
            const int n = counts[w * experts + e];
            counts[w * experts + e] = running;
            running += n;
        }
    }
    __syncthreads();
    int32_t* next = counts + wave * experts;    // this wave's running place for every expert; only this wave touches it
    for (int i0 = run0; i0 < run_end; i0 += 64) {
        const int i = i0 + lane;
        const int e = i < run_end ? chosen[i] : -1;
        unsigned long long left = __ballot(e >= 0);
        while (left) {
            const int leader = __ffsll((long long)left) - 1;
            const int expert = __shfl(e, leader, 64);
            const unsigned long long votes = __ballot(e == expert);
            const int first = next[expert];
            if (e == expert) {
                const int place = first + __popcll(votes & ((1ull << lane) - 1ull));
                place_row[place] = i / top;
                pair_place[i] = place;
            }
            if (lane == leader) next[expert] = first + __popcll(votes);
            left &= ~votes;
        }
    }
}

extern "C" int fw_moe_arrange(const int32_t* chosen, int32_t* expert_begin, int32_t* place_row, int32_t* pair_place, int rows, int experts,
                              int top, void* stream) {
    FW_REQUIRE(rows >= 0 && experts >= 1 && experts <= MOE_MAX_EXPERTS && top >= 1, "moe_arrange: bad sizes rows=%d experts=%d top=%d", rows, experts, top);
    FW_REQUIRE((long long)rows * top < (1ll << 30), "moe_arrange: too many pairs");
    const int lds_bytes = (MOE_ARRANGE_WAVES * experts + experts + 1) * (int)sizeof(int32_t);
    static int configured = 0;
    if (lds_bytes > 48 * 1024 && lds_bytes > configured) {
        hipError_t status = hipFuncSetAttribute((const void*)moe_arrange_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        FW_REQUIRE(status == hipSuccess, "moe_arrange: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(status));
        configured = lds_bytes;
    }
    moe_arrange_kernel<<<1, MOE_ARRANGE_THREADS, lds_bytes, (hipStream_t)stream>>>(chosen, expert_begin, place_row, pair_place, rows * top,
                                                                                  experts, top);
    FW_LAUNCH_CHECK("moe_arrange");
    return 0;
}

// The gated unit of a place: silu(gate) * up, or with a positive limit the clamped form
// g sigmoid(alpha g) (u + shift), g = min(gate, limit), u = clamp(up, -limit, limit).
struct GatedUnit {
    float limit, alpha, shift;
};
__device__ __forceinline__ float gg_clamped(float gate, float up, const GatedUnit unit) {
    const float g = fminf(gate, unit.limit), u = fminf(fmaxf(up, -unit.limit), unit.limit);
    return g / (1.0f + expf(-unit.alpha * g)) * (u + unit.shift);
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
                                                          TO* __restrict__ out, int experts, int N, int K, const GatedUnit unit) {
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
                value = unit.limit > 0.0f ? gg_clamped(g, acc[1][i][j], unit) : g / (1.0f + expf(-g)) * acc[1][i][j];
            }
            store_from_float(out, (size_t)(first + r) * N + col, value);
        }
    }
}

// ---- the grouped product on the matrix cores -----------------------------------------------------------
// bfloat16 operands, float32 accumulation (v_mfma_f32_32x32x16_bf16). A tile of places belongs to one
// expert; both operands are k-contiguous, a slab of 64 k of each is copied per iteration: global ->
// registers (two slabs ahead of the one multiplied) -> LDS (one ahead), two LDS buffers, one barrier an
// iteration, LDS rows padded to 144 bytes. Two shapes of tile:
//   BIG     128 places x 128 rows of W; four waves as 2 x 2, each 64 x 64. For steps in which an expert
//           has hundreds of places (prompts): the product is bound by the matrix cores.
//   small    32 places x (128 NJ) rows of W; four waves side by side, each 32 x (32 NJ). For steps of
//           few places an expert (decoding): the product is bound by how fast the experts' weights stream,
//           and every workgroup streams rows of W that no other reads.
// GATED: W is [2 N][K], gate rows then up rows; a tile takes as many gate rows as up rows of the same
// features, a wave holds gate and up of one element in one lane and stores silu(gate) * up.
// Which tile a workgroup has: an expert with n places has ceil(n / rows) tiles of places, each times the
// tiles of features; a wave finds its expert by a prefix sum of 64 experts' tile counts at a time. The grid
// holds as many tiles as there can be at most; a workgroup beyond the last leaves.
// A place's sum over k is formed in one order whatever the tile's shape and whoever shares the tile.
typedef __attribute__((ext_vector_type(8))) __bf16 gg_bf16x8;
typedef __attribute__((ext_vector_type(16))) float gg_f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t gg_u32x4;
#define GGM_TK 64
#define GGM_ROW_BYTES 144

__device__ __forceinline__ float gg_silu(float g) {
    if (g >= 0.0f) return g / (1.0f + __expf(-g));
    const float e = __expf(g);
    return g * e / (1.0f + e);
}

template <bool GATED, bool BIG, int NJ, typename TO>
__global__ __launch_bounds__(256) void grouped_gemm_mfma_kernel(
    const uint16_t* __restrict__ a, const int32_t* __restrict__ place_row, const uint16_t* __restrict__ w,
    const int32_t* __restrict__ expert_begin, TO* __restrict__ out, int experts, int N, int K, int tiles_m, int tiles_n, int per_xcd,
    const GatedUnit unit) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    constexpr int TMR = BIG ? 128 : 32;                 // places of a tile
    constexpr int WAVES_M = BIG ? 2 : 1, WAVES_N = 4 / WAVES_M;
    constexpr int NI = TMR / (32 * WAVES_M);
    constexpr int BN = WAVES_N * NJ * 32;               // rows of W of a tile
    constexpr int A_CHUNKS = TMR / 32, W_CHUNKS = BN / 32;
    constexpr int A_SLAB = TMR * GGM_ROW_BYTES, W_SLAB = BN * GGM_ROW_BYTES;
    static_assert(!GATED || NJ == 2, "the gated tile holds gate and up side by side");
    const int total = tiles_m * tiles_n;
    const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (logical >= total) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    // Workgroups are numbered expert by expert, within an expert feature tile by feature tile, and within that
    // over the expert's tiles of places: the two or three tiles that read the same rows of W run side by side,
    // and an expert's places (a megabyte or so) stay in the L2 of the XCD that works through the expert.
    int expert = -1, tile_in_expert = 0, pid_n = 0;
    {
        int before = 0;
        for (int e0 = 0; e0 < experts; e0 += 64) {
            const int e = e0 + lane;
            const int mine = e < experts ? (expert_begin[e + 1] - expert_begin[e] + TMR - 1) / TMR : 0;
            int upto = mine * tiles_n;
#pragma unroll
            for (int offset = 1; offset < 64; offset <<= 1) {
                const int other = __shfl_up(upto, offset, 64);
                if (lane >= offset) upto += other;
            }
            const unsigned long long holds = __ballot(logical < before + upto);
            if (holds) {
                const int at = __ffsll((long long)holds) - 1;
                const int tiles_here = __shfl(mine, at, 64);
                const int rest = logical - (before + __shfl(upto, at, 64) - tiles_here * tiles_n);
                expert = e0 + at;
                tile_in_expert = rest % tiles_here;
                pid_n = rest / tiles_here;
                break;
            }
            before += __shfl(upto, 63, 64);
        }
    }
    if (expert < 0) return;
    const int first = expert_begin[expert] + tile_in_expert * TMR, end = expert_begin[expert + 1];
    const int features = GATED ? BN / 2 : BN;
    const int n0 = pid_n * features;
    const int wm = BIG ? wave >> 1 : 0, wn = BIG ? wave & 1 : wave;
    const uint16_t* we = w + (size_t)expert * (GATED ? 2 : 1) * N * K;

    const uint16_t* a_src[A_CHUNKS];
    const uint16_t* w_src[W_CHUNKS];
    int a_at[A_CHUNKS], w_at[W_CHUNKS];
    const int kc = (tid & 7) * 8;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
        const int row = (tid >> 3) + 32 * i;
        int place = first + row;
        place = place < end ? place : end - 1;          // places past the expert's last are computed and dropped
        const int from = place_row ? place_row[place] : place;
        a_src[i] = a + (size_t)from * K;
        a_at[i] = row * GGM_ROW_BYTES + (tid & 7) * 16;
    }
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
        const int row = (tid >> 3) + 32 * i;
        int wr;
        if (GATED) {
            wr = row < BN / 2 ? n0 + row : n0 + row - BN / 2;
            wr = wr < N ? wr : N - 1;
            if (row >= BN / 2) wr += N;
        } else {
            wr = n0 + row;
            wr = wr < N ? wr : N - 1;
        }
        w_src[i] = we + (size_t)wr * K;
        w_at[i] = row * GGM_ROW_BYTES + (tid & 7) * 16;
    }

    gg_f32x16 acc[NI][NJ];
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    gg_u32x4 ra0[A_CHUNKS], rw0[W_CHUNKS], ra1[A_CHUNKS], rw1[W_CHUNKS];
    const gg_u32x4 zero = {0u, 0u, 0u, 0u};
    // Every load is issued unconditionally (past the end of K from column 0) and nothing touches the value
    // until it moves to LDS, so that the loads of two slabs stay in flight while a third is multiplied.
    auto fetch = [&](gg_u32x4 (&ra)[A_CHUNKS], gg_u32x4 (&rw)[W_CHUNKS], int k0) {
        const int from = k0 + kc < K ? k0 + kc : 0;     // K is a multiple of 8: columns 0..7 always exist
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) ra[i] = *reinterpret_cast<const gg_u32x4*>(a_src[i] + from);
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) rw[i] = *reinterpret_cast<const gg_u32x4*>(w_src[i] + from);
    };
    auto stash = [&](const gg_u32x4 (&ra)[A_CHUNKS], const gg_u32x4 (&rw)[W_CHUNKS], int buffer, int k0) {
        unsigned char* base = lds + buffer * (A_SLAB + W_SLAB);
        const bool ok = k0 + kc < K;                    // a past the end of K is zero; W may then be anything finite
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) *reinterpret_cast<gg_u32x4*>(base + a_at[i]) = ok ? ra[i] : zero;
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) *reinterpret_cast<gg_u32x4*>(base + A_SLAB + w_at[i]) = ok ? rw[i] : zero;
    };
    const int a_row0 = wm * 32 * NI + (lane & 31);
    int b_row[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
        b_row[j] = GATED ? j * (BN / 2) + wn * 32 + (lane & 31) : wn * (32 * NJ) + j * 32 + (lane & 31);
    const int k_lane = (lane >> 5) * 16;                // byte offset of this lane's 8 k within a k16 step
    auto multiply = [&](int buffer) {
        const unsigned char* sa = lds + buffer * (A_SLAB + W_SLAB);
        const unsigned char* sb = sa + A_SLAB;
#pragma unroll
        for (int k16 = 0; k16 < GGM_TK / 16; ++k16) {
            gg_bf16x8 fa[NI], fb[NJ];
#pragma unroll
            for (int i = 0; i < NI; ++i)
                fa[i] = *reinterpret_cast<const gg_bf16x8*>(sa + (a_row0 + 32 * i) * GGM_ROW_BYTES + k16 * 32 + k_lane);
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                fb[j] = *reinterpret_cast<const gg_bf16x8*>(sb + b_row[j] * GGM_ROW_BYTES + k16 * 32 + k_lane);
#pragma unroll
            for (int i = 0; i < NI; ++i)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
    };

    // slab s travels: global -> register set s % 2 (requested while slab s - 2 is multiplied) -> LDS buffer
    // s % 2 (stored while slab s - 1 is multiplied) -> multiplied
    const int steps = (K + GGM_TK - 1) / GGM_TK;
    int step = 0;
    fetch(ra0, rw0, 0);
    fetch(ra1, rw1, GGM_TK);                            // past the end: dropped when stored
    stash(ra0, rw0, 0, 0);
    fw_lds_barrier();
    while (step + 3 < steps) {
        fetch(ra0, rw0, (step + 2) * GGM_TK);
        __builtin_amdgcn_sched_barrier(0);              // keep the requests ahead of the work they overlap
        multiply(0);
        stash(ra1, rw1, 1, (step + 1) * GGM_TK);
        fw_lds_barrier();
        fetch(ra1, rw1, (step + 3) * GGM_TK);
        __builtin_amdgcn_sched_barrier(0);
        multiply(1);
        stash(ra0, rw0, 0, (step + 2) * GGM_TK);
        fw_lds_barrier();
        step += 2;
    }
    // at most three slabs are left: slab `step` is in buffer 0, slab step + 1 in set 1
    if (step + 2 < steps) fetch(ra0, rw0, (step + 2) * GGM_TK);
    multiply(0);
    if (step + 1 < steps) {
        stash(ra1, rw1, 1, (step + 1) * GGM_TK);
        fw_lds_barrier();
        multiply(1);
        if (step + 2 < steps) {
            stash(ra0, rw0, 0, (step + 2) * GGM_TK);
            fw_lds_barrier();
            multiply(0);
        }
    }
    fw_mfma_drain();     // the branches below lead to code that reads the accumulators

    // D layout of the 32x32 product: lane holds column lane % 32; register r is row 8 * (r / 4) + 4 * (lane / 32) + r % 4
    const int col = lane & 31, row_base = (lane >> 5) * 4;
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int place = first + wm * 32 * NI + i * 32 + 8 * (r >> 2) + row_base + (r & 3);
            if (place >= end) continue;
            if (GATED) {
                const int n = n0 + wn * 32 + col;
                if (n < N)
                    store_from_float(out, (size_t)place * N + n, unit.limit > 0.0f ? gg_clamped(acc[i][0][r], acc[i][NJ - 1][r], unit)
                                                                                    : gg_silu(acc[i][0][r]) * acc[i][NJ - 1][r]);
            } else {
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    const int n = n0 + wn * (32 * NJ) + j * 32 + col;
                    if (n < N) store_from_float(out, (size_t)place * N + n, acc[i][j][r]);
                }
            }
        }
}

template <bool GATED, bool BIG, int NJ, typename TO>
static int grouped_mfma_launch(const void* a, const int32_t* place_row, const void* w, const int32_t* expert_begin, void* out, int places,
                               int experts, int N, int K, const GatedUnit unit, hipStream_t stream) {
    constexpr int TMR = BIG ? 128 : 32;
    constexpr int BN = (BIG ? 2 : 4) * NJ * 32;
    const int features = GATED ? BN / 2 : BN;
    const long long tiles_m = (long long)places / TMR + (experts < places ? experts : places);    // at most
    const long long tiles_n = fw_ceil_div(N, features);
    FW_REQUIRE(tiles_m * tiles_n < (1ll << 30), "grouped_gemm: too many tiles");
    const int per_xcd = (int)fw_ceil_div(tiles_m * tiles_n, 8);
    const int lds_bytes = 2 * (TMR + BN) * GGM_ROW_BYTES;
    static bool configured = false;     // per instantiation
    if (!configured) {
        hipError_t status = hipFuncSetAttribute((const void*)grouped_gemm_mfma_kernel<GATED, BIG, NJ, TO>,
                                                hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        FW_REQUIRE(status == hipSuccess, "grouped_gemm: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(status));
        configured = true;
    }
    grouped_gemm_mfma_kernel<GATED, BIG, NJ, TO><<<per_xcd * 8, 256, lds_bytes, stream>>>(
        (const uint16_t*)a, place_row, (const uint16_t*)w, expert_begin, (TO*)out, experts, N, K, (int)tiles_m, (int)tiles_n, per_xcd, unit);
    return 0;
}

extern "C" int fw_grouped_gemm(const void* a, int a_dtype, const int32_t* place_row, const void* w, int w_dtype,
                               const int32_t* expert_begin, void* out, int out_dtype, int gated, int places, int experts, int N, int K,
                               float glu_limit, float glu_alpha, float glu_shift, void* stream) {
    const GatedUnit unit = {glu_limit, glu_alpha, glu_shift};
    FW_REQUIRE(glu_limit <= 0.0f || gated, "grouped_gemm: a clamped unit goes with gate and up rows");
    FW_REQUIRE(places >= 0 && experts >= 1 && N > 0 && K > 0, "grouped_gemm: bad sizes places=%d experts=%d N=%d K=%d", places, experts, N, K);
    if (places == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    // bfloat16 operands go to the matrix cores: tiles of 128 places where experts have many, of 32 where few
    if (a_dtype == FW_BF16 && w_dtype == FW_BF16 && K % 8 == 0 && (uintptr_t)a % 16 == 0 && (uintptr_t)w % 16 == 0 &&
        (out_dtype == FW_F32 || (out_dtype == FW_BF16 && gated))) {
        const bool big = (long long)places >= 48ll * experts;
        int status;
        if (gated) status = big ? grouped_mfma_launch<true, true, 2, bf16_t>(a, place_row, w, expert_begin, out, places, experts, N, K, unit, s)
                                : grouped_mfma_launch<true, false, 2, bf16_t>(a, place_row, w, expert_begin, out, places, experts, N, K, unit, s);
        else status = big ? grouped_mfma_launch<false, true, 2, float>(a, place_row, w, expert_begin, out, places, experts, N, K, unit, s)
                          : grouped_mfma_launch<false, false, 1, float>(a, place_row, w, expert_begin, out, places, experts, N, K, unit, s);
        if (status != 0) return status;
        FW_LAUNCH_CHECK("grouped_gemm");
        return 0;
    }
    const long long tiles = (long long)places / GG_ROWS + experts;      // at most: every expert may end in a tile that is not full
    FW_REQUIRE(tiles < (1ll << 31) && (N + GG_COLS - 1) / GG_COLS <= 65535, "grouped_gemm: grid too large");
    dim3 grid((unsigned)tiles, (N + GG_COLS - 1) / GG_COLS);
#define FW_GG_LAUNCH(TA, TW, TO)                                                                                                   \
    {                                                                                                                              \
        if (gated) grouped_gemm_kernel<TA, TW, TO, true><<<grid, 256, 0, s>>>((const TA*)a, place_row, (const TW*)w, expert_begin, \
                                                                              (TO*)out, experts, N, K, unit);                     \
        else grouped_gemm_kernel<TA, TW, TO, false><<<grid, 256, 0, s>>>((const TA*)a, place_row, (const TW*)w, expert_begin,      \
                                                                         (TO*)out, experts, N, K, unit);                          \
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
