// A feed-forward of many small gated experts of which every token uses a few.
//
//   route      s = sigmoid(z) for float32 router logits z [tokens, experts]; the `top` largest are chosen, ranked
//              by z itself (s rises with z, but two large z can round to one s; the lowest index wins a tie);
//              a (token, choice) *pair* p = token * top + k gets the expert and the score as it is (not
//              renormalised).
//   arrange    pairs sorted by expert and cut into tiles of at most `tile_rows` rows of one expert; everything the
//              later kernels need stays on the device (the count of tiles too), so a step can be captured: grids
//              are sized for the most tiles there can be, and workgroups past the count leave at once.
//   gate_up    act[i, :] = glu(W_gate[e] (w x), W_up[e] (w x)) for the i-th sorted pair: the pair's weight w
//              multiplies the expert's *input* row x (the unit is not linear, so it cannot move to the output).
//   down       parts[p, :] = W_down[e] act[i, :], float32, one row per pair: whoever adds the branch sums a
//              token's `top` rows, in a fixed order.
//
// bfloat16 with widths that are multiples of 8 runs on the matrix cores, in one of two forms.  Few rows an expert (a
// decode step): four waves a workgroup, each a tile of 16 columns over all of K for up to 16 * RT rows, operands
// straight from memory.  Many rows an expert (a prompt's portion): the rows are first gathered in sorted order and
// multiplied by their weights (`gather`), then tiles of 128 rows x 128 columns a workgroup, slices of 64 k staged
// through LDS in the operand order of the matrix instruction, the next slice's loads under way while this one is
// multiplied.  Anything else takes the plain form of one thread per result, whose sums run over k in order, float32.  Weights: gate_up [experts, 2 * ff, hidden] (gate rows first), down
// [experts, hidden, ff].
#include "activation_forms.h"
#include "attention_args.h"
#include "common.h"

using cie_attention::bf16x8;
using cie_attention::floatx4;

namespace {

constexpr int kMaxExperts = 1024;

// How a token's router outputs become a choice and weights.  Every step may be left out:
//   s = sigmoid(z), or softmax(z) over all outputs                        (softmax)
//   the choice ranks c = s + correction[e]                                (correction; without one and without the
//                                                                          softmax the logits z themselves are ranked)
//   the outputs form `groups` equal runs of neighbours; a run's score is its largest c, and only outputs of the
//   `keep` best runs can be chosen                                        (groups > 1)
//   weights w = s of the chosen, as they are, or divided by their sum + 1e-20 and times `scale`   (normalize)
struct RouteShape {
    int softmax;
    const float* correction;  // [outputs] or null
    int groups;               // <= 1: none (at most 64)
    int keep;
    int normalize;
    float scale;
};

// One wave ranks one token's logits z: its `top` outputs and their weights to expert_out / weight_out (and the
// outputs to `copy` as well, where the caller wants them in LDS).  Equal ranks: the lower index first.
__device__ __forceinline__ void route_token(const float* __restrict__ z, int experts, int top, int lane,
                                            int* __restrict__ expert_out, float* __restrict__ weight_out,
                                            int* copy, const RouteShape shape) {
    constexpr int kMine = kMaxExperts / kWave;
    float mine[kMine];   // what is ranked
    float score[kMine];  // what becomes the weight
    unsigned out = 0;  // bit i: expert lane + i * kWave is not there, or already chosen, or outside the kept runs
    float z_max = -INFINITY;
#pragma unroll
    for (int i = 0; i < kMine; ++i) {
        const int e = lane + i * kWave;
        mine[i] = e < experts ? z[e] : 0.f;  // (ranked by the logit: the score rises with it, and does not saturate)
        if (e >= experts) out |= 1u << i;
        else z_max = fmaxf(z_max, mine[i]);
    }
    const bool by_score = shape.softmax || shape.correction;
    if (shape.softmax) {
        z_max = wave_max(z_max);
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < kMine; ++i) {
            score[i] = (lane + i * kWave < experts) ? expf(mine[i] - z_max) : 0.f;
            sum += score[i];
        }
        const float inv = 1.0f / wave_sum(sum);
#pragma unroll
        for (int i = 0; i < kMine; ++i) score[i] *= inv;
    } else {
#pragma unroll
        for (int i = 0; i < kMine; ++i) score[i] = 1.0f / (1.0f + expf(-mine[i]));
    }
    if (by_score) {
#pragma unroll
        for (int i = 0; i < kMine; ++i) {
            const int e = lane + i * kWave;
            mine[i] = score[i] + ((shape.correction && e < experts) ? shape.correction[e] : 0.f);
        }
    }
    if (shape.groups > 1) {
        // lane g holds run g's score; then the `keep` best runs, one after the other
        const int per = experts / shape.groups;
        float run_score = -INFINITY;
        for (int g = 0; g < shape.groups; ++g) {
            float best = -INFINITY;
#pragma unroll
            for (int i = 0; i < kMine; ++i) {
                const int e = lane + i * kWave;
                if (e < experts && e / per == g) best = fmaxf(best, mine[i]);
            }
            best = wave_max(best);
            if (lane == g) run_score = best;
        }
        unsigned long long kept = 0;
        for (int k = 0; k < shape.keep; ++k) {
            float best = run_score;
            int best_g = (lane < shape.groups && !((kept >> lane) & 1ull)) ? lane : kWave;
#pragma unroll
            for (int offset = kWave / 2; offset > 0; offset >>= 1) {
                const float other = __shfl_xor(best, offset, kWave);
                const int other_g = __shfl_xor(best_g, offset, kWave);
                if (other_g != kWave && (best_g == kWave || other > best || (other == best && other_g < best_g))) {
                    best = other;
                    best_g = other_g;
                }
            }
            if (best_g != kWave) kept |= 1ull << best_g;
        }
#pragma unroll
        for (int i = 0; i < kMine; ++i) {
            const int e = lane + i * kWave;
            if (e < experts && !((kept >> (e / per)) & 1ull)) out |= 1u << i;
        }
    }
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
        float best = 0.f;
        int best_e = kMaxExperts;  // (none yet)
#pragma unroll
        for (int i = 0; i < kMine; ++i) {
            // (ascending index within the lane: the first of equals stays)
            if (!((out >> i) & 1u) && (best_e == kMaxExperts || mine[i] > best)) {
                best = mine[i];
                best_e = lane + i * kWave;
            }
        }
#pragma unroll
        for (int offset = kWave / 2; offset > 0; offset >>= 1) {
            const float other = __shfl_xor(best, offset, kWave);
            const int other_e = __shfl_xor(best_e, offset, kWave);
            if (other_e != kMaxExperts &&
                (best_e == kMaxExperts || other > best || (other == best && other_e < best_e))) {
                best = other;
                best_e = other_e;
            }
        }
        float chosen = 0.f;  // the score of the chosen one, from the lane that holds it
#pragma unroll
        for (int i = 0; i < kMine; ++i)
            if (lane + i * kWave == best_e) {
                out |= 1u << i;
                chosen = score[i];
            }
        chosen = __shfl(chosen, best_e % kWave, kWave);
        total += chosen;
        if (lane == 0) {
            expert_out[k] = best_e;
            weight_out[k] = chosen;
            if (copy) copy[k] = best_e;
        }
    }
    if (shape.normalize && lane == 0) {
        const float factor = shape.scale / (total + 1e-20f);
        for (int k = 0; k < top; ++k) weight_out[k] *= factor;  // (this thread's own stores)
    }
}

// One wave per token.
__global__ void __launch_bounds__(256)
route_kernel(const float* __restrict__ logits, int tokens, int experts, int top, int* __restrict__ pair_expert,
             float* __restrict__ pair_weight, RouteShape shape) {
    const int lane = threadIdx.x % kWave;
    const int token = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
    if (token >= tokens) return;
    route_token(logits + static_cast<size_t>(token) * experts, experts, top, lane,
                pair_expert + static_cast<size_t>(token) * top, pair_weight + static_cast<size_t>(token) * top, nullptr,
                shape);
}

// One workgroup.  sorted[i]: the pair at place i of the order by expert; tiles (expert, first place, rows).
// (pair_expert may lie in LDS.)  Only the first `real` of the `experts` router outputs have weights and get tiles:
// the pairs of the others stand at the end of the order, and whoever owns them fills their rows.
__device__ __forceinline__ void arrange_pairs(const int* pair_expert, int pairs, int experts, int real, int tile_rows,
                                              int* __restrict__ sorted, int* __restrict__ tile_expert,
                                              int* __restrict__ tile_begin, int* __restrict__ tile_count,
                                              int* __restrict__ n_tiles) {
    __shared__ int count[kMaxExperts];
    __shared__ int first[kMaxExperts];
    __shared__ int first_tile[kMaxExperts];
    __shared__ int cursor[kMaxExperts];
    for (int e = threadIdx.x; e < experts; e += blockDim.x) {
        count[e] = 0;
        cursor[e] = 0;
    }
    __syncthreads();
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) atomicAdd(&count[pair_expert[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int place = 0, tile = 0;
        for (int e = 0; e < experts; ++e) {
            first[e] = place;
            first_tile[e] = tile;
            place += count[e];
            if (e < real) tile += (count[e] + tile_rows - 1) / tile_rows;
        }
        *n_tiles = tile;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < real; e += blockDim.x) {
        const int tiles = (count[e] + tile_rows - 1) / tile_rows;
        for (int t = 0; t < tiles; ++t) {
            tile_expert[first_tile[e] + t] = e;
            tile_begin[first_tile[e] + t] = first[e] + t * tile_rows;
            tile_count[first_tile[e] + t] = min(tile_rows, count[e] - t * tile_rows);
        }
    }
    // (the order of an expert's pairs among themselves follows the order of arrival: every row is computed
    //  by itself, so no result depends on it)
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        const int e = pair_expert[p];
        sorted[first[e] + atomicAdd(&cursor[e], 1)] = p;
    }
}

__global__ void __launch_bounds__(1024)
arrange_kernel(const int* __restrict__ pair_expert, int pairs, int experts, int real, int tile_rows,
               int* __restrict__ sorted, int* __restrict__ tile_expert, int* __restrict__ tile_begin,
               int* __restrict__ tile_count, int* __restrict__ n_tiles) {
    arrange_pairs(pair_expert, pairs, experts, real, tile_rows, sorted, tile_expert, tile_begin, tile_count, n_tiles);
}

// Few tokens (a step of up to sixteen single tokens): choice and order in one workgroup, one launch (beyond that
// the waves would rank several tokens one after the other, and two launches are faster).  A wave ranks every
// sixteenth token; the chosen experts wait in LDS for the ordering.
constexpr int kFusedPairs = 1024;
constexpr int kFusedTokens = 16;

__global__ void __launch_bounds__(1024)
route_arrange_kernel(const float* __restrict__ logits, int tokens, int experts, int real, int top,
                     int* __restrict__ pair_expert, float* __restrict__ pair_weight, int tile_rows,
                     int* __restrict__ sorted, int* __restrict__ tile_expert, int* __restrict__ tile_begin,
                     int* __restrict__ tile_count, int* __restrict__ n_tiles, RouteShape shape) {
    __shared__ int chosen[kFusedPairs];
    const int lane = threadIdx.x % kWave;
    for (int token = threadIdx.x / kWave; token < tokens; token += blockDim.x / kWave)
        route_token(logits + static_cast<size_t>(token) * experts, experts, top, lane,
                    pair_expert + static_cast<size_t>(token) * top, pair_weight + static_cast<size_t>(token) * top,
                    chosen + token * top, shape);
    __syncthreads();
    arrange_pairs(chosen, tokens * top, experts, real, tile_rows, sorted, tile_expert, tile_begin, tile_count, n_tiles);
}

struct ExpertArgs {
    const int* sorted;
    const float* pair_weight;
    const int* tile_expert;
    const int* tile_begin;
    const int* tile_count;
    const int* n_tiles;
    int top;
    int hidden;
    int ff;
    float limit;
    float alpha;
    float offset;
};

__device__ __forceinline__ bf16x8 scaled_fragment(const uint4 raw, float w) {
    const uint32_t v[4] = {raw.x, raw.y, raw.z, raw.w};
    uint32_t out[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        out[i] = pack_bf16(__uint_as_float(v[i] << 16) * w, __uint_as_float(v[i] & 0xffff0000u) * w);
    return __builtin_bit_cast(bf16x8, (uint4{out[0], out[1], out[2], out[3]}));
}

// v_mfma_f32_16x16x32_bf16 with A = rows of x (lane % 16 the row, lane / 16 the eighth of the 32 k), B = rows of
// the weight (lane % 16 the result column, the same k): lane (r, g) then holds the results of rows g*4 .. g*4+3 at
// column r.
// Loads stand without conditions (addresses past an edge are clamped, what they fetch is zeroed when used), the loads
// of kUnroll steps of 32 k ahead of the products that use them: a wave has that many cache lines of its weight rows
// under way at once, which is what a step of few rows, bound by the weights' way from memory, needs.
constexpr int kUnroll = 4;

// SPLIT: the tiles are few (a step of a few single tokens), and a wave per 16 columns would leave most SIMDs idle:
// the workgroup's four waves share 16 columns, each takes a quarter of K, and the quarters meet in LDS, summed in
// the waves' order.
template <int RT, bool SPLIT>
__global__ void __launch_bounds__(256)
experts_gate_up_mfma_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w_gate_up,
                            bf16_t* __restrict__ act, ExpertArgs a) {
    __shared__ float meet[SPLIT ? 3 * 2 * RT * 4 * kWave : 1];
    const int tile = blockIdx.x;
    if (tile >= *a.n_tiles) return;
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int r = lane & 15;
    const int g = lane >> 4;
    const int c0 = SPLIT ? blockIdx.y * 16 : (blockIdx.y * 4 + wave) * 16;
    if (c0 >= a.ff) return;
    const int expert = a.tile_expert[tile];
    const int begin = a.tile_begin[tile];
    const int rows = a.tile_count[tile];
    const int K = a.hidden;
    const bool col_ok = c0 + r < a.ff;
    const bf16_t* wg = w_gate_up + (static_cast<size_t>(expert) * 2 * a.ff + min(c0 + r, a.ff - 1)) * K;
    const bf16_t* wu = wg + static_cast<size_t>(a.ff) * K;
    const bf16_t* x_row[RT];
    float weight[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int row = rt * 16 + r;
        const int pair = a.sorted[begin + min(row, rows - 1)];
        x_row[rt] = x + static_cast<size_t>(pair / a.top) * K;
        weight[rt] = row < rows ? (a.pair_weight ? a.pair_weight[pair] : 1.f) : 0.f;
    }
    floatx4 acc_g[RT], acc_u[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) acc_g[rt] = acc_u[rt] = floatx4{0.f, 0.f, 0.f, 0.f};
    const int quarter = ((K + 3) / 4 + 7) & ~7;                 // (pieces of 8 k stay whole)
    const int k_begin = SPLIT ? wave * quarter : 0;
    const int k_end = SPLIT ? min(K, k_begin + quarter) : K;
    for (int k0 = k_begin; k0 < k_end; k0 += 32 * kUnroll) {
        uint4 bg[kUnroll], bu[kUnroll], ax[kUnroll][RT];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int k = min(k0 + u * 32 + g * 8, K - 8);
            bg[u] = *reinterpret_cast<const uint4*>(wg + k);
            bu[u] = *reinterpret_cast<const uint4*>(wu + k);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) ax[u][rt] = *reinterpret_cast<const uint4*>(x_row[rt] + k);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const bool k_ok = k0 + u * 32 + g * 8 < k_end;
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                const bf16x8 af = scaled_fragment(ax[u][rt], k_ok ? weight[rt] : 0.f);
                acc_g[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, __builtin_bit_cast(bf16x8, bg[u]), acc_g[rt], 0, 0, 0);
                acc_u[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, __builtin_bit_cast(bf16x8, bu[u]), acc_u[rt], 0, 0, 0);
            }
        }
    }
    if (SPLIT) {
        // meet[wave - 1][gate | up][rt][i][lane]
        if (wave > 0) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    meet[(((wave - 1) * 2 + 0) * RT + rt) * 4 * kWave + i * kWave + lane] = acc_g[rt][i];
                    meet[(((wave - 1) * 2 + 1) * RT + rt) * 4 * kWave + i * kWave + lane] = acc_u[rt][i];
                }
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int w = 0; w < 3; ++w)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc_g[rt][i] += meet[((w * 2 + 0) * RT + rt) * 4 * kWave + i * kWave + lane];
                    acc_u[rt][i] += meet[((w * 2 + 1) * RT + rt) * 4 * kWave + i * kWave + lane];
                }
    }
    if (!col_ok) return;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = rt * 16 + g * 4 + i;
            if (row < rows)
                act[static_cast<size_t>(begin + row) * a.ff + c0 + r] =
                    from_float<bf16_t>(clamped_glu(acc_g[rt][i], acc_u[rt][i], a.limit, a.alpha, a.offset));
        }
}

template <int RT, bool SPLIT>
__global__ void __launch_bounds__(256)
experts_down_mfma_kernel(const bf16_t* __restrict__ act, const bf16_t* __restrict__ w_down, float* __restrict__ parts,
                         ExpertArgs a) {
    __shared__ float meet[SPLIT ? 3 * RT * 4 * kWave : 1];
    const int tile = blockIdx.x;
    if (tile >= *a.n_tiles) return;
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int r = lane & 15;
    const int g = lane >> 4;
    const int c0 = SPLIT ? blockIdx.y * 16 : (blockIdx.y * 4 + wave) * 16;
    if (c0 >= a.hidden) return;
    const int expert = a.tile_expert[tile];
    const int begin = a.tile_begin[tile];
    const int rows = a.tile_count[tile];
    const int K = a.ff;
    const bool col_ok = c0 + r < a.hidden;
    const bf16_t* wd = w_down + (static_cast<size_t>(expert) * a.hidden + min(c0 + r, a.hidden - 1)) * K;
    const bf16_t* a_row[RT];
    bool row_ok[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        row_ok[rt] = rt * 16 + r < rows;
        a_row[rt] = act + static_cast<size_t>(begin + min(rt * 16 + r, rows - 1)) * K;
    }
    floatx4 acc[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) acc[rt] = floatx4{0.f, 0.f, 0.f, 0.f};
    const uint4 zero = uint4{0, 0, 0, 0};
    const int quarter = ((K + 3) / 4 + 7) & ~7;
    const int k_begin = SPLIT ? wave * quarter : 0;
    const int k_end = SPLIT ? min(K, k_begin + quarter) : K;
    for (int k0 = k_begin; k0 < k_end; k0 += 32 * kUnroll) {
        uint4 b[kUnroll], ax[kUnroll][RT];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int k = min(k0 + u * 32 + g * 8, K - 8);
            b[u] = *reinterpret_cast<const uint4*>(wd + k);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) ax[u][rt] = *reinterpret_cast<const uint4*>(a_row[rt] + k);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const bool k_ok = k0 + u * 32 + g * 8 < k_end;
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                const uint4 raw = (k_ok && row_ok[rt]) ? ax[u][rt] : zero;
                acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, raw),
                                                                  __builtin_bit_cast(bf16x8, b[u]), acc[rt], 0, 0, 0);
            }
        }
    }
    if (SPLIT) {
        if (wave > 0) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int i = 0; i < 4; ++i) meet[((wave - 1) * RT + rt) * 4 * kWave + i * kWave + lane] = acc[rt][i];
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int w = 0; w < 3; ++w)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[rt][i] += meet[(w * RT + rt) * 4 * kWave + i * kWave + lane];
    }
    if (!col_ok) return;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = rt * 16 + g * 4 + i;
            if (row < rows) parts[static_cast<size_t>(a.sorted[begin + row]) * a.hidden + c0 + r] = acc[rt][i];
        }
}


// ---- many rows an expert: tiles of 128 x 128 through LDS ---------------------------------------------------------
// A slice of 64 k of 128 operand rows lies in LDS as [128 rows][8 pieces of 8 k], piece p of row m at place
// p ^ ((m >> 1) & 7) of the row: the sixteen lanes that the hardware serves together then touch every bank once, both
// when a matrix instruction's operand is read (rows m .. m + 15, one piece) and when a slice is staged (two rows,
// all their pieces; a thread stages 16 bytes of rows t / 8 + 32 j, which it fetched as whole cache lines a row).
// Wave w of four owns rows 64 (w / 2) .. and the column half w % 2: 4 x 4 products of 16 x 16 per 32 k.
constexpr int kTile = 128;
constexpr int kSlice = 64;
constexpr int kXcds = 8;

// xs[i, :] = bf16(weight(pair) * x[token(pair), :]) for the i-th pair of the sorted order.
__global__ void __launch_bounds__(256)
experts_gather_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ xs, const int* __restrict__ sorted,
                      const float* __restrict__ pair_weight, int pairs, int top, int hidden) {
    const int place = blockIdx.x;
    const int pair = sorted[place];
    const float w = pair_weight ? pair_weight[pair] : 1.f;
    const bf16_t* src = x + static_cast<size_t>(pair / top) * hidden;
    bf16_t* dst = xs + static_cast<size_t>(place) * hidden;
    for (int k = threadIdx.x * 8; k < hidden; k += blockDim.x * 8) {
        const uint4 raw = *reinterpret_cast<const uint4*>(src + k);
        *reinterpret_cast<uint4*>(dst + k) = __builtin_bit_cast(uint4, scaled_fragment(raw, w));
    }
}

// GATE_UP: a[rows, K] x (gate rows | up rows of 64 result columns) -> act = unit(gate, up), bfloat16.
// else:    a[rows, K] x 128 rows of the down weight -> parts[pair], float32.
template <bool GATE_UP>
__global__ void __launch_bounds__(256)
experts_tiled_kernel(const bf16_t* __restrict__ a_rows, const bf16_t* __restrict__ weight, bf16_t* __restrict__ act,
                     float* __restrict__ parts, ExpertArgs a) {
    __shared__ __attribute__((aligned(16))) bf16_t lds_a[2][kTile * kSlice];
    __shared__ __attribute__((aligned(16))) bf16_t lds_b[2][kTile * kSlice];
    const int K = GATE_UP ? a.hidden : a.ff;
    const int n_out = GATE_UP ? a.ff : a.hidden;            // result columns of the expert
    const int cols_here = GATE_UP ? kTile / 2 : kTile;      // ... of which this workgroup makes so many
    // Workgroup b of a launch goes to XCD b % 8, and each XCD has an L2 of its own.  An XCD takes a run of
    // neighbouring tiles (tiles are in the order of their experts) and walks it column block by column block: the
    // workgroups that are in flight on it together share a few tiles' rows and, where neighbouring tiles are one
    // expert's, that expert's weights.
    const int n_tiles = *a.n_tiles;
    const int col_blocks = (n_out + cols_here - 1) / cols_here;
    const int per_xcd = (n_tiles + kXcds - 1) / kXcds;
    const int turn = blockIdx.x / kXcds;
    const int tile = (blockIdx.x % kXcds) * per_xcd + turn / col_blocks;
    if (turn / col_blocks >= per_xcd || tile >= n_tiles) return;
    const int c0 = (turn % col_blocks) * cols_here;
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int r = lane & 15;
    const int g = lane >> 4;
    const int expert = a.tile_expert[tile];
    const int begin = a.tile_begin[tile];
    const int rows = a.tile_count[tile];
    // staging: thread t brings 16 bytes (8 k) of rows t / 8 + 32 j, j = 0..3, for A and for B
    const int s_row = threadIdx.x / 8;
    const int s_k = (threadIdx.x % 8) * 8;
    const bf16_t* a_src[4];
    const bf16_t* b_src[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int row = s_row + 32 * j;
        a_src[j] = a_rows + static_cast<size_t>(begin + min(row, rows - 1)) * K;
        // weight row of staged row `row`: GATE_UP lays the workgroup's columns out as [half][gate 32 | up 32]
        int col;
        if (GATE_UP) {
            const int half = row / 64, within = row % 64;
            col = c0 + half * 32 + (within % 32);
            col = min(col, n_out - 1) + (within >= 32 ? n_out : 0);
        } else {
            col = min(c0 + row, n_out - 1);
        }
        b_src[j] = weight + (static_cast<size_t>(expert) * (GATE_UP ? 2 * n_out : n_out) + col) * K;
    }
    auto place = [](int row, int piece) { return row * kSlice + ((piece ^ ((row >> 1) & 7)) << 3); };
    // Two sets of registers hold the slices that are on their way: set 0 the even ones, set 1 the odd ones.  While
    // slice s is multiplied, slices s + 1 and s + 2 are under way, so a load has two slices' products to arrive in
    // (one was not enough: the matrix cores take a slice faster than the L2 answers under this traffic).  The sets
    // are vector values with names of their own and the steps are macros: arrays of structs that are handed to a
    // function by reference, or indexed by a loop's counter, went through scratch memory.
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    u32x4 ra0[4], rb0[4], ra1[4], rb1[4];
#define CIE_FETCH(fa, fb, k0_)                                                                                   \
    {                                                                                                            \
        const int k_ = min((k0_) + s_k, K - 8); /* (past K: clamped, and what it brings is never multiplied) */  \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                                          \
            fa[j] = *reinterpret_cast<const u32x4*>(a_src[j] + k_);                                              \
            fb[j] = *reinterpret_cast<const u32x4*>(b_src[j] + k_);                                              \
        }                                                                                                        \
    }
#define CIE_STAGE(buffer_, fa, fb, k0_)                                                                          \
    {                                                                                                            \
        const bool k_ok_ = (k0_) + s_k < K; /* (a slice past the end of K holds zeros on the A side) */          \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                                          \
            const int at_ = place(s_row + 32 * j, s_k >> 3);                                                     \
            *reinterpret_cast<u32x4*>(&lds_a[buffer_][at_]) = k_ok_ ? fa[j] : u32x4{0, 0, 0, 0};                 \
            *reinterpret_cast<u32x4*>(&lds_b[buffer_][at_]) = fb[j];                                             \
        }                                                                                                        \
    }
#define CIE_MULTIPLY(buffer_)                                                                                    \
    _Pragma("unroll") for (int half = 0; half < 2; ++half) {                                                     \
        bf16x8 af[4], bfr[4];                                                                                    \
        _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                                          \
            af[i] = *reinterpret_cast<const bf16x8*>(&lds_a[buffer_][place(row0 + i * 16 + r, half * 4 + g)]);   \
            bfr[i] = *reinterpret_cast<const bf16x8*>(&lds_b[buffer_][place(col0 + i * 16 + r, half * 4 + g)]);  \
        }                                                                                                        \
        _Pragma("unroll") for (int i = 0; i < 4; ++i)                                                            \
            _Pragma("unroll") for (int j = 0; j < 4; ++j)                                                        \
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);          \
    }
    floatx4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
    const int row0 = (wave / 2) * 64;
    const int col0 = (wave % 2) * 64;
    CIE_FETCH(ra0, rb0, 0);
    CIE_STAGE(0, ra0, rb0, 0);
    CIE_FETCH(ra1, rb1, kSlice);
    __syncthreads();
    for (int k0 = 0; k0 < K; k0 += 2 * kSlice) {
        CIE_FETCH(ra0, rb0, k0 + 2 * kSlice);
        CIE_MULTIPLY(0);
        if (k0 + kSlice < K) CIE_STAGE(1, ra1, rb1, k0 + kSlice);
        __syncthreads();
        if (k0 + kSlice < K) {
            CIE_FETCH(ra1, rb1, k0 + 3 * kSlice);
            CIE_MULTIPLY(1);
            if (k0 + 2 * kSlice < K) CIE_STAGE(0, ra0, rb0, k0 + 2 * kSlice);
            __syncthreads();
        }
    }
#undef CIE_FETCH
#undef CIE_STAGE
#undef CIE_MULTIPLY
    // lane (r, g) holds rows g*4 .. g*4+3 of row tile i at column r of column tile j
    if (GATE_UP) {
        // the wave's 64 staged columns are [gate 32 | up 32] of result columns c0 + (wave % 2) * 32 ..
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int col = c0 + (wave % 2) * 32 + j * 16 + r;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int row = row0 + i * 16 + g * 4 + v;
                    if (row < rows && col < n_out)
                        act[static_cast<size_t>(begin + row) * n_out + col] =
                            from_float<bf16_t>(clamped_glu(acc[i][j][v], acc[i][j + 2][v], a.limit, a.alpha, a.offset));
                }
            }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int row = row0 + i * 16 + g * 4 + v;
                if (row >= rows) continue;
                float* dst = parts + static_cast<size_t>(a.sorted[begin + row]) * n_out;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int col = c0 + col0 + j * 16 + r;
                    if (col < n_out) dst[col] = acc[i][j][v];
                }
            }
    }
}

// The plain forms: tiles of up to 16 rows, 16 columns a workgroup, one thread per result.
template <typename T>
__global__ void __launch_bounds__(256)
experts_gate_up_plain_kernel(const T* __restrict__ x, const T* __restrict__ w_gate_up, T* __restrict__ act, ExpertArgs a) {
    const int tile = blockIdx.x;
    if (tile >= *a.n_tiles) return;
    const int row = threadIdx.x / 16;
    const int col = blockIdx.y * 16 + threadIdx.x % 16;
    if (row >= a.tile_count[tile] || col >= a.ff) return;
    const int expert = a.tile_expert[tile];
    const int place = a.tile_begin[tile] + row;
    const int pair = a.sorted[place];
    const float w = a.pair_weight ? a.pair_weight[pair] : 1.f;
    const int K = a.hidden;
    const T* x_row = x + static_cast<size_t>(pair / a.top) * K;
    const T* wg = w_gate_up + (static_cast<size_t>(expert) * 2 * a.ff + col) * K;
    const T* wu = wg + static_cast<size_t>(a.ff) * K;
    float sum_g = 0.f, sum_u = 0.f;
    for (int k = 0; k < K; ++k) {
        const float v = to_float(from_float<T>(to_float(x_row[k]) * w));  // the scaled input, as the storage type holds it
        sum_g = fmaf(v, to_float(wg[k]), sum_g);
        sum_u = fmaf(v, to_float(wu[k]), sum_u);
    }
    act[static_cast<size_t>(place) * a.ff + col] = from_float<T>(clamped_glu(sum_g, sum_u, a.limit, a.alpha, a.offset));
}

template <typename T>
__global__ void __launch_bounds__(256)
experts_down_plain_kernel(const T* __restrict__ act, const T* __restrict__ w_down, float* __restrict__ parts, ExpertArgs a) {
    const int tile = blockIdx.x;
    if (tile >= *a.n_tiles) return;
    const int row = threadIdx.x / 16;
    const int col = blockIdx.y * 16 + threadIdx.x % 16;
    if (row >= a.tile_count[tile] || col >= a.hidden) return;
    const int expert = a.tile_expert[tile];
    const int place = a.tile_begin[tile] + row;
    const int K = a.ff;
    const T* a_row = act + static_cast<size_t>(place) * K;
    const T* wd = w_down + (static_cast<size_t>(expert) * a.hidden + col) * K;
    float sum = 0.f;
    for (int k = 0; k < K; ++k) sum = fmaf(to_float(a_row[k]), to_float(wd[k]), sum);
    parts[static_cast<size_t>(a.sorted[place]) * a.hidden + col] = sum;
}

// parts[p, :] = x[token(p), :] for every pair whose choice is one of the outputs behind the `real` experts (an
// expert that hands its input on); the other pairs' rows are the down product's.
template <typename T>
__global__ void __launch_bounds__(256)
experts_identity_kernel(const T* __restrict__ x, const int* __restrict__ pair_expert, int real,
                        float* __restrict__ parts, int top, int hidden) {
    const int pair = blockIdx.x;
    if (pair_expert[pair] < real) return;
    const T* src = x + static_cast<size_t>(pair / top) * hidden;
    float* dst = parts + static_cast<size_t>(pair) * hidden;
    for (int k = threadIdx.x; k < hidden; k += blockDim.x) dst[k] = to_float(src[k]);
}

}  // namespace

CIE_API int cie_experts_identity(void* stream, int dtype, const void* x, const int* pair_expert, int real, float* parts,
                                 int pairs, int top, int hidden) {
    if (pairs < 0 || top < 1 || hidden < 1 || real < 0) return CIE_BAD_ARGUMENT;
    if (pairs == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == CIE_F32)
        experts_identity_kernel<float><<<pairs, 256, 0, s>>>(static_cast<const float*>(x), pair_expert, real, parts, top, hidden);
    else if (dtype == CIE_BF16)
        experts_identity_kernel<bf16_t><<<pairs, 256, 0, s>>>(static_cast<const bf16_t*>(x), pair_expert, real, parts, top, hidden);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}

// `experts` router outputs of which the first `real` are experts with weights (the others hand their input on: their
// pairs get no tiles).  The choice's shape: see RouteShape.
CIE_API int cie_experts_route(void* stream, const float* logits, int tokens, int experts, int top, int tile_rows,
                              int* pair_expert, float* pair_weight, int* sorted, int* tile_expert, int* tile_begin,
                              int* tile_count, int* n_tiles, int real, int softmax, const float* correction,
                              int groups, int keep, int normalize, float scale) {
    if (tokens < 0 || experts < 1 || experts > kMaxExperts || top < 1 || top > experts || tile_rows < 1 || real < 0 ||
        real > experts)
        return CIE_BAD_ARGUMENT;
    if (groups > 1 && (groups > kWave || experts % groups || keep < 1 || keep > groups || top > keep * (experts / groups)))
        return CIE_BAD_ARGUMENT;
    const RouteShape shape{softmax, correction, groups, keep, normalize, scale};
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (tokens > 0 && tokens <= kFusedTokens && tokens * top <= kFusedPairs) {
        route_arrange_kernel<<<1, 1024, 0, s>>>(logits, tokens, experts, real, top, pair_expert, pair_weight, tile_rows,
                                                sorted, tile_expert, tile_begin, tile_count, n_tiles, shape);
        return cie_after_launch();
    }
    if (tokens > 0) {
        route_kernel<<<(tokens + 3) / 4, 256, 0, s>>>(logits, tokens, experts, top, pair_expert, pair_weight, shape);
        if (hipGetLastError() != hipSuccess) return CIE_LAUNCH_FAILED;
    }
    arrange_kernel<<<1, 1024, 0, s>>>(pair_expert, tokens * top, experts, real, tile_rows, sorted, tile_expert,
                                      tile_begin, tile_count, n_tiles);
    return cie_after_launch();
}

// A wave per 16 result columns of every tile there can be: fewer waves than the chip has SIMDs (256 compute units of
// four) take the form that splits K over a workgroup's waves.
static bool few_waves(int max_tiles, int columns) {
    return static_cast<long>(max_tiles) * ((columns + 15) / 16) <= 1024;
}

// act [pairs, ff] in the storage type, rows in sorted order.  `mfma` != 0: the matrix-core form (bfloat16, hidden
// and ff multiples of 8, tile_rows 16 * row_tiles with row_tiles 1, 2 or 4); else tile_rows must be <= 16.
CIE_API int cie_experts_gate_up(void* stream, int dtype, int mfma, const void* x, const void* w_gate_up, void* act,
                                const int* sorted, const float* pair_weight, const int* tile_expert,
                                const int* tile_begin, const int* tile_count, const int* n_tiles, int max_tiles,
                                int tile_rows, int top, int hidden, int ff, float limit, float alpha, float offset) {
    if (max_tiles < 0 || top < 1 || hidden < 1 || ff < 1 || !(limit > 0.f) || tile_rows < 1) return CIE_BAD_ARGUMENT;
    if (max_tiles == 0) return CIE_OK;
    const ExpertArgs a{sorted, pair_weight, tile_expert, tile_begin, tile_count, n_tiles, top, hidden, ff, limit, alpha, offset};
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (mfma) {
        if (dtype != CIE_BF16 || hidden % 8 || ff % 8) return CIE_BAD_ARGUMENT;
        dim3 grid(max_tiles, (ff + 63) / 64);
        const bf16_t* xs = static_cast<const bf16_t*>(x);
        const bf16_t* ws = static_cast<const bf16_t*>(w_gate_up);
        bf16_t* as = static_cast<bf16_t*>(act);
        if (tile_rows == kTile) {  // (x: the rows gathered in sorted order, weights applied)
            experts_tiled_kernel<true><<<kXcds * ((max_tiles + kXcds - 1) / kXcds) * ((ff + 63) / 64), 256, 0, s>>>(xs, ws, as, nullptr, a);
            return cie_after_launch();
        }
        if (tile_rows == 16 && few_waves(max_tiles, ff))
            experts_gate_up_mfma_kernel<1, true><<<dim3(max_tiles, (ff + 15) / 16), 256, 0, s>>>(xs, ws, as, a);
        else if (tile_rows == 16) experts_gate_up_mfma_kernel<1, false><<<grid, 256, 0, s>>>(xs, ws, as, a);
        else if (tile_rows == 32) experts_gate_up_mfma_kernel<2, false><<<grid, 256, 0, s>>>(xs, ws, as, a);
        else if (tile_rows == 64) experts_gate_up_mfma_kernel<4, false><<<grid, 256, 0, s>>>(xs, ws, as, a);
        else return CIE_BAD_ARGUMENT;
        return cie_after_launch();
    }
    if (tile_rows > 16) return CIE_BAD_ARGUMENT;
    dim3 grid(max_tiles, (ff + 15) / 16);
    if (dtype == CIE_F32)
        experts_gate_up_plain_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(x), static_cast<const float*>(w_gate_up),
                                                                static_cast<float*>(act), a);
    else if (dtype == CIE_BF16)
        experts_gate_up_plain_kernel<bf16_t><<<grid, 256, 0, s>>>(static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w_gate_up),
                                                                 static_cast<bf16_t*>(act), a);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}

// parts [pairs, hidden] float32, row p the pair p = token * top + k.
CIE_API int cie_experts_down(void* stream, int dtype, int mfma, const void* act, const void* w_down, float* parts,
                             const int* sorted, const int* tile_expert, const int* tile_begin, const int* tile_count,
                             const int* n_tiles, int max_tiles, int tile_rows, int top, int hidden, int ff) {
    if (max_tiles < 0 || top < 1 || hidden < 1 || ff < 1 || tile_rows < 1) return CIE_BAD_ARGUMENT;
    if (max_tiles == 0) return CIE_OK;
    const ExpertArgs a{sorted, nullptr, tile_expert, tile_begin, tile_count, n_tiles, top, hidden, ff, 1.f, 1.f, 0.f};
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (mfma) {
        if (dtype != CIE_BF16 || hidden % 8 || ff % 8) return CIE_BAD_ARGUMENT;
        dim3 grid(max_tiles, (hidden + 63) / 64);
        const bf16_t* as = static_cast<const bf16_t*>(act);
        const bf16_t* ws = static_cast<const bf16_t*>(w_down);
        if (tile_rows == kTile) {
            experts_tiled_kernel<false><<<kXcds * ((max_tiles + kXcds - 1) / kXcds) * ((hidden + kTile - 1) / kTile), 256, 0, s>>>(as, ws, nullptr, parts, a);
            return cie_after_launch();
        }
        if (tile_rows == 16 && few_waves(max_tiles, hidden))
            experts_down_mfma_kernel<1, true><<<dim3(max_tiles, (hidden + 15) / 16), 256, 0, s>>>(as, ws, parts, a);
        else if (tile_rows == 16) experts_down_mfma_kernel<1, false><<<grid, 256, 0, s>>>(as, ws, parts, a);
        else if (tile_rows == 32) experts_down_mfma_kernel<2, false><<<grid, 256, 0, s>>>(as, ws, parts, a);
        else if (tile_rows == 64) experts_down_mfma_kernel<4, false><<<grid, 256, 0, s>>>(as, ws, parts, a);
        else return CIE_BAD_ARGUMENT;
        return cie_after_launch();
    }
    if (tile_rows > 16) return CIE_BAD_ARGUMENT;
    dim3 grid(max_tiles, (hidden + 15) / 16);
    if (dtype == CIE_F32)
        experts_down_plain_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(act), static_cast<const float*>(w_down), parts, a);
    else if (dtype == CIE_BF16)
        experts_down_plain_kernel<bf16_t><<<grid, 256, 0, s>>>(static_cast<const bf16_t*>(act), static_cast<const bf16_t*>(w_down), parts, a);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}

// xs [pairs, hidden]: row i is the input row of the i-th sorted pair times the pair's weight (bfloat16, hidden a
// multiple of 8): what the tiled form of cie_experts_gate_up takes as x.
CIE_API int cie_experts_gather(void* stream, const void* x, void* xs, const int* sorted, const float* pair_weight,
                               int pairs, int top, int hidden) {
    if (pairs < 0 || top < 1 || hidden < 8 || hidden % 8) return CIE_BAD_ARGUMENT;
    if (pairs == 0) return CIE_OK;
    experts_gather_kernel<<<pairs, 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const bf16_t*>(x), static_cast<bf16_t*>(xs), sorted, pair_weight, pairs, top, hidden);
    return cie_after_launch();
}
