// Paged grouped-query attention whose scores are shaped before the softmax, and the kernel that prepares its
// heads.  Every shaping step is a parameter and may be left out:
//
//   s_ij = (q_i . k_j) * scale
//   s_ij <- cap * tanh(s_ij / cap)                       cap > 0
//   s_ij <- s_ij - slope[head] * (i - j)                 slopes given (a bias on the distance itself)
//   j is seen by i when 0 <= i - j < window              window > 0 (else every j <= i)
//   ... or, beside the window, when j < keep <= ...       keep > 0: the first `keep` keys of the sequence stay visible
//                                                        to every later token, at their own positions
//   ... or when j <= i and floor(i / chunk) = floor(j / chunk)   chunk > 0: chunks counted from position 0
//   p_ij = exp(s_ij) / (sum_j exp(s_ij) + exp(sink[head]))   sinks given: one more term in the denominator, which
//                                                        has no key and no value, no scale and no bias
//   o_i  = sum_j p_ij v_j,  o_i <- o_i * sigmoid(gate[i, head])   gate given
//
// Keys have D numbers per head, values DV (the two may differ).  Cache layout as everywhere in this library:
// keys [pages, kv_heads, page_size, D], values transposed [pages, kv_heads, DV, page_size].  Scores, the softmax,
// the value sums and the gate are float32 in both storage types.
//
// `cie_heads_prepare` is what stands between the projection and this attention: a per-head RMS norm of queries
// and keys (with a weight, without one, or none; or one RMS norm over all query heads of a token together and one
// over all its key heads, with a weight per number of the projection), the queries' factor that grows with the position,
//   q <- q * (1 + coef * ln(floor((p + 1) / every) + 1)),
// then a rotation of the first `rot` numbers of every query and key head by the position (pairs of neighbours or of
// the two halves; cos and sin from float32 tables [positions, rot / 2]),
// queries laid out [tokens, heads, D] (zero-padded from the projection's head size up to D) and keys and values
// written to the cache (padded likewise).  Statistics, the logarithm and the scaling are float32.
#include "attention_args.h"
#include "common.h"

using namespace cie_attention;

namespace {

// ------------------------------------------------------------------------------------------------ prepare
// A wave's sum of the squares of n numbers: sixteen bytes a lane and load where the numbers start at a multiple of
// sixteen bytes (every wave of a token sums the whole projection again under the norm over all heads: the loads
// are what that costs).
__device__ __forceinline__ float wave_sum_squares(const float* p, int n, int lane) {
    float sum = 0.f;
    int done = 0;
    if ((reinterpret_cast<uintptr_t>(p) & 15) == 0) {
        for (int d = 4 * lane; d + 3 < n; d += 4 * kWave) {
            const float4 v = *reinterpret_cast<const float4*>(p + d);
            sum += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
        }
        done = n & ~3;
    }
    for (int d = done + lane; d < n; d += kWave) sum += p[d] * p[d];
    return wave_sum(sum);
}
__device__ __forceinline__ float wave_sum_squares(const bf16_t* p, int n, int lane) {
    float sum = 0.f;
    int done = 0;
    if ((reinterpret_cast<uintptr_t>(p) & 15) == 0) {
        for (int d = 8 * lane; d + 7 < n; d += 8 * kWave) {
            const uint4 raw = *reinterpret_cast<const uint4*>(p + d);
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float lo = __uint_as_float(w[i] << 16), hi = __uint_as_float(w[i] & 0xffff0000u);
                sum += lo * lo + hi * hi;
            }
        }
        done = n & ~7;
    }
    for (int d = done + lane; d < n; d += kWave) {
        const float x = to_float(p[d]);
        sum += x * x;
    }
    return wave_sum(sum);
}

// One wave per (token, head slot): slots 0..H-1 queries, H..H+G-1 keys, H+G..H+2G-1 values.
template <typename T>
__global__ void __launch_bounds__(256)
heads_prepare_kernel(const T* __restrict__ proj, int proj_stride, int q_off, int k_off, int v_off,
                     const float* __restrict__ q_weight, const float* __restrict__ k_weight, int norm_mode,
                     float eps, float temp_coef, int temp_every, const int* __restrict__ positions,
                     const int* __restrict__ seq_of_token, const int* __restrict__ seq_slot,
                     const int* __restrict__ block_table, int table_width, T* __restrict__ q_out,
                     T* __restrict__ k_pool, T* __restrict__ v_pool, int tokens, int q_heads, int kv_heads,
                     int dim, int vdim, int D, int DV, int page_shift, int write_kv,
                     const float* __restrict__ cos_table, const float* __restrict__ sin_table, int rot, int neighbours) {
    const int lane = threadIdx.x % kWave;
    const int slots = q_heads + 2 * kv_heads;
    const long unit = static_cast<long>(blockIdx.x) * (blockDim.x / kWave) + threadIdx.x / kWave;
    if (unit >= static_cast<long>(tokens) * slots) return;
    const int token = static_cast<int>(unit / slots);
    const int slot = static_cast<int>(unit - static_cast<long>(token) * slots);
    const int pos = positions[token];
    const T* row = proj + static_cast<size_t>(token) * proj_stride;
    const int page_size = 1 << page_shift;
    size_t page = 0;
    if (slot >= q_heads) {
        if (!write_kv) return;
        const int* table = block_table + static_cast<size_t>(seq_slot[seq_of_token[token]]) * table_width;
        page = static_cast<size_t>(table[pos >> page_shift]);
    }
    if (slot >= q_heads + kv_heads) {  // a value head: copied, padded, into the transposed pool
        const int head = slot - q_heads - kv_heads;
        const T* src = row + v_off + head * vdim;
        T* dst = v_pool + ((page * kv_heads + head) * DV << page_shift) + (pos & (page_size - 1));
        for (int d = lane; d < DV; d += kWave)
            dst[static_cast<size_t>(d) << page_shift] = d < vdim ? src[d] : from_float<T>(0.f);
        return;
    }
    const bool is_q = slot < q_heads;
    const int head = is_q ? slot : slot - q_heads;
    const T* src = row + (is_q ? q_off : k_off) + head * dim;
    const float* weight = is_q ? q_weight : k_weight;
    float factor = 1.f;
    if (norm_mode == 3) {  // one root mean square over all heads of the projection; the weight has a number for each
        const int all = (is_q ? q_heads : kv_heads) * dim;
        const T* whole = row + (is_q ? q_off : k_off);
        factor = 1.0f / sqrtf(wave_sum_squares(whole, all, lane) / static_cast<float>(all) + eps);
        weight += head * dim;
    } else if (norm_mode != 0) {
        float sum_sq = 0.f;
        for (int d = lane; d < dim; d += kWave) {
            const float x = to_float(src[d]);
            sum_sq += x * x;
        }
        factor = 1.0f / sqrtf(wave_sum(sum_sq) / static_cast<float>(dim) + eps);
    }
    const bool weighted = norm_mode >= 2;
    float after = 1.f;  // the queries' factor of the position
    if (is_q && temp_every > 0)
        after = 1.0f + temp_coef * logf(static_cast<float>((pos + 1) / temp_every) + 1.0f);
    T* dst = is_q ? q_out + (static_cast<size_t>(token) * q_heads + head) * D
                  : k_pool + (((page * kv_heads + head) << page_shift) + (pos & (page_size - 1))) * D;
    const int half = rot / 2;
    const float* cos_row = rot > 0 ? cos_table + static_cast<size_t>(pos) * half : nullptr;
    const float* sin_row = rot > 0 ? sin_table + static_cast<size_t>(pos) * half : nullptr;
    for (int d = lane; d < D; d += kWave) {
        float x = 0.f;
        if (d < dim) {
            x = to_float(src[d]) * factor;
            if (weighted) x *= weight[d];
            if (d < rot) {
                // the pair (u, v) of the angle's index i turns to (u cos - v sin, v cos + u sin): neighbours
                // (2i, 2i + 1) or the halves (i, i + rot / 2)
                const int i = neighbours ? d >> 1 : (d < half ? d : d - half);
                const bool is_u = neighbours ? !(d & 1) : d < half;
                const int mate = neighbours ? d ^ 1 : (is_u ? d + half : d - half);
                float y = to_float(src[mate]) * factor;
                if (weighted) y *= weight[mate];
                const float c = cos_row[i], sn = sin_row[i];
                x = is_u ? x * c - y * sn : x * c + y * sn;
            }
            x *= after;
        }
        dst[d] = from_float<T>(x);
    }
}

// ------------------------------------------------------------------------------------------------ generic
// One workgroup (4 waves) per (query token, query head); each wave takes 64-key chunks in turn, one key per
// lane for the scores, then one slice of the value head per lane; the four running (max, sum, accumulator)
// triples meet in LDS.  Any D, DV that are multiples of 8 up to 256; float32 or bfloat16 storage.
constexpr int kMaxSlices = 4;

template <typename T>
__device__ __forceinline__ void load8(const T* p, float (&v)[8]);
template <>
__device__ __forceinline__ void load8<float>(const float* p, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    const float4 b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
template <>
__device__ __forceinline__ void load8<bf16_t>(const bf16_t* p, float (&v)[8]) {
    const uint4 raw = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(w[i] << 16);
        v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}

struct ScoreShape {
    float scale;
    float softcap;        // <= 0: none
    const float* slopes;  // [q_heads] or null
    const float* sinks;   // [q_heads] or null
    int window;           // <= 0: all keys
    int chunk;            // > 0: i sees j <= i only inside its own chunk, floor(i / chunk) == floor(j / chunk)
    int keep;             // > 0 (with a window): keys 0 .. keep - 1 are seen from behind the window too
};

// The first key that the query at position `pos` sees.
__device__ __forceinline__ int first_seen(int pos, int window, int chunk) {
    if (chunk > 0) return pos < 0 ? 0 : pos - pos % chunk;
    return window > 0 ? max(0, pos + 1 - window) : 0;
}

template <typename T>
__global__ void __launch_bounds__(256)
scored_attention_generic_kernel(const T* __restrict__ q, const T* __restrict__ k_pool, const T* __restrict__ v_pool,
                                const int* __restrict__ block_table, int table_width,
                                const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                                const int* __restrict__ seq_slot, const T* __restrict__ gate, int gate_stride,
                                T* __restrict__ out, int q_heads, int kv_heads, int D, int DV, int page_size,
                                ScoreShape shape) {
    extern __shared__ float lds[];
    float* q_s = lds;            // [D]
    float* acc_s = lds + D;      // [4][DV]
    __shared__ float m_s[4];
    __shared__ float l_s[4];

    const int token = blockIdx.x;
    const int head = blockIdx.y;
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int kv_head = head / (q_heads / kv_heads);
    const int pos = positions[token];
    const int len = pos + 1;
    const int lo = first_seen(pos, shape.window, shape.chunk);
    const int* table = block_table + static_cast<size_t>(seq_slot[seq_of_token[token]]) * table_width;
    const float slope = shape.slopes ? shape.slopes[head] : 0.f;

    const T* q_row = q + (static_cast<size_t>(token) * q_heads + head) * D;
    for (int d = threadIdx.x; d < D; d += blockDim.x) q_s[d] = to_float(q_row[d]);
    __syncthreads();

    float m = -INFINITY;
    float l = 0.f;
    float acc[kMaxSlices] = {0.f, 0.f, 0.f, 0.f};
    // the keys in the order they are walked: the kept first ones that lie in front of the window, then the window's
    const int kept = (shape.window > 0 && shape.keep > 0) ? min(shape.keep, lo) : 0;
    const int walk = kept + len - lo;
    for (int base = wave * kWave; base < walk; base += 4 * kWave) {
        const int at = base + lane;
        const int key = at < kept ? at : at - kept + lo;
        const bool valid = at < walk;
        float s = -INFINITY;
        uint32_t head_block = 0;
        uint32_t in_page = 0;
        if (valid) {
            const int page = table[key / page_size];
            head_block = static_cast<uint32_t>(page) * kv_heads + kv_head;
            in_page = key % page_size;
            const T* k_row = k_pool + (static_cast<size_t>(head_block) * page_size + in_page) * D;
            float dot = 0.f;
            for (int d = 0; d < D; d += 8) {
                float kk[8];
                load8<T>(k_row + d, kk);
#pragma unroll
                for (int j = 0; j < 8; ++j) dot = fmaf(q_s[d + j], kk[j], dot);
            }
            s = dot * shape.scale;
            if (shape.softcap > 0.f) s = shape.softcap * tanhf(s / shape.softcap);
            s -= slope * static_cast<float>(pos - key);
        }
        const float m_new = fmaxf(m, wave_max(s));  // finite: lane 0 of every chunk is valid
        const float alpha = expf(m - m_new);
        const float p = valid ? expf(s - m_new) : 0.f;
        l = l * alpha + wave_sum(p);
#pragma unroll
        for (int i = 0; i < kMaxSlices; ++i) acc[i] *= alpha;
        const int count = min(kWave, walk - base);
        for (int j = 0; j < count; ++j) {
            const float pj = __shfl(p, j, kWave);
            const uint32_t block_j = __shfl(head_block, j, kWave);
            const uint32_t in_page_j = __shfl(in_page, j, kWave);
            const T* v_column = v_pool + static_cast<size_t>(block_j) * page_size * DV + in_page_j;
#pragma unroll
            for (int i = 0; i < kMaxSlices; ++i) {
                const int d = lane + kWave * i;
                if (d < DV) acc[i] = fmaf(pj, to_float(v_column[static_cast<size_t>(d) * page_size]), acc[i]);
            }
        }
        m = m_new;
    }
    if (lane == 0) {
        m_s[wave] = m;
        l_s[wave] = l;
    }
#pragma unroll
    for (int i = 0; i < kMaxSlices; ++i) {
        const int d = lane + kWave * i;
        if (d < DV) acc_s[wave * DV + d] = acc[i];
    }
    __syncthreads();
    float m_all = m_s[0];
    for (int w = 1; w < 4; ++w) m_all = fmaxf(m_all, m_s[w]);
    const float sink = shape.sinks ? shape.sinks[head] : -INFINITY;
    m_all = fmaxf(m_all, sink);
    float den = shape.sinks ? expf(sink - m_all) : 0.f;
    float e[4];
    for (int w = 0; w < 4; ++w) {
        e[w] = expf(m_s[w] - m_all);  // a wave that saw no key has m = -inf: weight 0
        den += l_s[w] * e[w];
    }
    float open = 1.f;
    if (gate) open = 1.0f / (1.0f + expf(-to_float(gate[static_cast<size_t>(token) * gate_stride + head])));
    T* out_row = out + (static_cast<size_t>(token) * q_heads + head) * DV;
    for (int d = threadIdx.x; d < DV; d += blockDim.x) {
        float num = 0.f;
        for (int w = 0; w < 4; ++w) num += acc_s[w * DV + d] * e[w];
        out_row[d] = from_float<T>(num / den * open);
    }
}

// ------------------------------------------------------------------------------------------------ matrix cores
// bfloat16.  A workgroup of four waves per (tile, kv head); a tile is up to `tokens_per_tile` consecutive query
// tokens of one sequence, its rows the (token, head of the group) pairs: row = token * G + head, at most 16 * RT.
// Wave w takes every fourth block of 32 keys of the range the tile can see, so each key and value is read once
// per workgroup.  Per block, as in the other matrix-core attention kernels of this library:
//   S^T[key, row] = K[key, :] . Q[row, :]   v_mfma_f32_16x16x32_bf16, A = K, B = Q; lane (r = lane % 16,
//   g = lane / 16) then holds, for row r, the scores of keys g*4 .. g*4+3 of each 16-key tile, which is the A-operand
//   layout of P in  O[row, d] += P[row, key] * V[key, d]  (B = rows of the transposed values).
// The softmax runs in base 2 (scores, cap, bias and sink are brought there once).  The four waves' running
// (max, sum, accumulator) meet in LDS, one wave after the other, and all threads write the tile's rows.  Few tiles
// over many keys (single tokens behind long windows) have their keys cut into shares, a workgroup each, whose
// (max, sum, accumulator) a second kernel joins; sink and gate are then applied there.  The accumulator is rescaled
// only in blocks where some row's maximum moved, and keys are masked only in blocks that reach an edge of some row.
struct ScoredArgs {
    const bf16_t* q;          // [tokens, q_heads, D]
    const bf16_t* k_pool;
    const bf16_t* v_pool;
    const int* block_table;
    int table_width;
    const int* tile_seq;      // null: tile i is the first tile of sequence i
    const int* tile_q0;
    const int* seq_slot;
    const int* seq_start;
    const int* seq_q_len;
    const int* q_start_loc;
    const bf16_t* gate;       // [tokens, gate_stride], column = head; or null
    int gate_stride;
    bf16_t* out;              // [tokens, q_heads, DV]
    int q_heads;
    int kv_heads;
    int page_shift;
    int tokens_per_tile;
    int n_tiles;
    int n_splits;        // > 1: the keys of a tile in that many shares of keys_per_split (a multiple of 128), one
    int keys_per_split;  // workgroup each (blockIdx.z); the shares' sums meet in scored_attention_merge_kernel
    float* part_o;       // [tiles, kv_heads, splits, rows, DV]
    float* part_ml;      // [tiles, kv_heads, splits, rows, 2]
    ScoreShape shape;
};

constexpr int kScoredWaves = 4;
constexpr float kLog2e = 1.44269504088896341f;

__device__ __forceinline__ float fast_tanh(float y) {
    // tanh(y) = 1 - 2 / (exp(2y) + 1); exp through the hardware's base-2 exponential
    const float e = __builtin_amdgcn_exp2f(fminf(y * (2.f * kLog2e), 126.f));
    return 1.f - 2.f * __builtin_amdgcn_rcpf(e + 1.f);
}

template <int D, int DV, int RT>
__global__ void __launch_bounds__(64 * kScoredWaves, RT <= 2 ? 2 : 1) scored_attention_mfma_kernel(ScoredArgs a) {
    constexpr int NK = D / 32;
    constexpr int ND = DV / 16;
    constexpr int ROWS = 16 * RT;
    constexpr int STEP = kKeysPerBlock * kScoredWaves;
    __shared__ float m_s[kScoredWaves][ROWS];
    __shared__ float l_s[kScoredWaves][ROWS];
    __shared__ float o_s[ROWS][DV + 1];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int r = lane & 15;
    const int g = lane >> 4;
    const int tile = a.n_tiles - 1 - static_cast<int>(blockIdx.x);  // the last tiles of a prompt see the most keys
    const int kv_head = blockIdx.y;
    const int group = a.q_heads / a.kv_heads;
    const int seq = a.tile_seq ? a.tile_seq[tile] : tile;
    const int q0 = a.tile_seq ? a.tile_q0[tile] : 0;
    const int start = a.seq_start[seq];
    const int n_tok = min(a.tokens_per_tile, a.seq_q_len[seq] - q0);
    const int n_rows = n_tok * group;
    const int first_row_token = a.q_start_loc[seq] + q0;
    const int page_mask = (1 << a.page_shift) - 1;
    const int* table = a.block_table + static_cast<size_t>(a.seq_slot[seq]) * a.table_width;
    const float scale = a.shape.scale;
    const float cap = a.shape.softcap;
    const float inv_cap = cap > 0.f ? 1.0f / cap : 0.f;
    const int window = a.shape.window;

    const int hi = start + q0 + n_tok;
    const int chunk = a.shape.chunk;
    const int lo = first_seen(start + q0, window, chunk);
    // The blocks of keys are walked in an order of their own: with kept first keys that lie wholly in front of the
    // window's first block, blocks 0 .. kept_span - 1 come first and the window's blocks follow them; a walked index at
    // or beyond kept_span is `gap` keys short of the key it stands for.  Otherwise walked index and key are the same.
    const int keep = (window > 0 && a.shape.keep > 0) ? a.shape.keep : 0;
    int range_begin = lo & ~(kKeysPerBlock - 1);
    int kept_span = 0, gap = 0;
    if (keep > 0) {
        const int kept_blocks = (min(keep, hi) + kKeysPerBlock - 1) & ~(kKeysPerBlock - 1);
        if (kept_blocks < range_begin) {
            kept_span = kept_blocks;
            gap = range_begin - kept_blocks;
        }
        range_begin = 0;
    }
    int range_end = hi - gap;
    const int split = blockIdx.z;
    if (a.n_splits > 1) {
        range_begin += split * a.keys_per_split;
        range_end = min(hi - gap, range_begin + a.keys_per_split);
    }
    const int first_pos = start + q0;            // position of the tile's first token (its window reaches back furthest)
    const int last_lo = first_seen(start + q0 + n_tok - 1, window, chunk);  // the first key the tile's last token sees

    if (a.n_splits > 1 && range_begin >= range_end) {  // a share without keys: its statistics say so, its sums are never read
        float* pml = a.part_ml + ((static_cast<size_t>(tile) * a.kv_heads + kv_head) * a.n_splits + split) * ROWS * 2;
        if (threadIdx.x < ROWS) {
            pml[threadIdx.x * 2] = -INFINITY;
            pml[threadIdx.x * 2 + 1] = 0.f;
        }
        return;
    }

    uint4 qf[RT][NK];
    int row_pos[RT];      // position of the lane's row r of tile rt; -1 for a row that does not exist
    float row_slope[RT];  // its head's slope, in base-2 units
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int row = rt * 16 + r;
        const bool valid = row < n_rows;
        const int tok = valid ? row / group : 0;
        const int head = kv_head * group + (valid ? row - tok * group : 0);
        row_pos[rt] = valid ? start + q0 + tok : -1;
        row_slope[rt] = a.shape.slopes ? a.shape.slopes[head] * kLog2e : 0.f;
        const bf16_t* q_row = a.q + (static_cast<size_t>(first_row_token + tok) * a.q_heads + head) * D + g * (D / 4);
#pragma unroll
        for (int j = 0; j < NK; ++j)
            qf[rt][j] = valid ? *reinterpret_cast<const uint4*>(q_row + j * 8) : uint4{0, 0, 0, 0};
    }

    float m_run[RT], l_run[RT];
    floatx4 o[RT][ND];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        m_run[rt] = -INFINITY;
        l_run[rt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) o[rt][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    for (int at = range_begin + wave * kKeysPerBlock; at < range_end; at += STEP) {
        const int kb = at < kept_span ? at : at + gap;  // the block's first key
        const int block_end = range_end + (kb - at);    // where this share's keys end, counted in keys of this block's stretch
        // every row sees every key of the block: none lies behind the first token, none before the last one's window
        // (or all are kept first keys)
        const bool inner = kb + kKeysPerBlock - 1 <= first_pos && (kb >= last_lo || kb + kKeysPerBlock <= keep) &&
                           kb + kKeysPerBlock <= block_end;
        floatx4 s[RT][2];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            const int key = min(kb + kt * 16 + r, hi - 1);  // keys past the end are masked below
            const int page = table[key >> a.page_shift];
            const bf16_t* k_row = a.k_pool +
                (((static_cast<size_t>(page) * a.kv_heads + kv_head) << a.page_shift) + (key & page_mask)) * D +
                g * (D / 4);
            uint4 kf[NK];
#pragma unroll
            for (int j = 0; j < NK; ++j) kf[j] = *reinterpret_cast<const uint4*>(k_row + j * 8);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < NK; ++j)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf[j]),
                                                                  __builtin_bit_cast(bf16x8, qf[rt][j]), acc, 0, 0, 0);
                s[rt][kt] = acc;
            }
        }
        uint2 vf[ND][2];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            const int key = min(kb + kt * 16 + g * 4, (hi - 1) & ~3);
            const int page = table[key >> a.page_shift];
            const bf16_t* v_base = a.v_pool +
                ((static_cast<size_t>(page) * a.kv_heads + kv_head) * DV << a.page_shift) + (key & page_mask);
#pragma unroll
            for (int dt = 0; dt < ND; ++dt)
                vf[dt][kt] = *reinterpret_cast<const uint2*>(v_base + (static_cast<size_t>(dt * 16 + r) << a.page_shift));
        }
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            const int pos = row_pos[rt];
            const int row_lo = first_seen(pos, window, chunk);
            float block_max = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = kb + kt * 16 + g * 4 + i;
                    const bool seen = inner || (key <= pos && (key >= row_lo || key < keep) && key < block_end);
                    float x = s[rt][kt][i] * scale;
                    if (cap > 0.f) x = cap * fast_tanh(x * inv_cap);
                    x = x * kLog2e - row_slope[rt] * static_cast<float>(pos - key);
                    x = seen ? x : -INFINITY;
                    s[rt][kt][i] = x;
                    block_max = fmaxf(block_max, x);
                }
            }
            block_max = fmaxf(block_max, __shfl_xor(block_max, 16, kWave));
            block_max = fmaxf(block_max, __shfl_xor(block_max, 32, kWave));
            const float m_new = fmaxf(m_run[rt], block_max);
            const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m_run[rt] - m_safe);  // m_run = -inf: 0, and l, O are 0 anyway
            const bool moved = m_new != m_run[rt];
            m_run[rt] = m_new;
            float p_sum = 0.f;
            uint32_t pw[4];
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
                const float p0 = __builtin_amdgcn_exp2f(s[rt][kt][0] - m_safe);
                const float p1 = __builtin_amdgcn_exp2f(s[rt][kt][1] - m_safe);
                const float p2 = __builtin_amdgcn_exp2f(s[rt][kt][2] - m_safe);
                const float p3 = __builtin_amdgcn_exp2f(s[rt][kt][3] - m_safe);
                p_sum += (p0 + p1) + (p2 + p3);
                pw[kt * 2] = pack_bf16(p0, p1);
                pw[kt * 2 + 1] = pack_bf16(p2, p3);
            }
            l_run[rt] = l_run[rt] * alpha + p_sum;
            if (__any(moved)) {
                // the accumulator's rows are g*4+i, the statistics' row is r: fetch alpha of those rows
                float alpha_o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) alpha_o[i] = __shfl(alpha, g * 4 + i, kWave);
#pragma unroll
                for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) o[rt][dt][i] *= alpha_o[i];
            }
            const bf16x8 p_frag = __builtin_bit_cast(bf16x8, (uint4{pw[0], pw[1], pw[2], pw[3]}));
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) {
                const uint4 v = uint4{vf[dt][0].x, vf[dt][0].y, vf[dt][1].x, vf[dt][1].y};
                o[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(p_frag, __builtin_bit_cast(bf16x8, v), o[rt][dt], 0, 0, 0);
            }
        }
    }

    // ---- the waves' statistics, then the common reference of every row and the whole denominator
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        float l = l_run[rt];
        l += __shfl_xor(l, 16, kWave);
        l += __shfl_xor(l, 32, kWave);
        if (g == 0) {
            m_s[wave][rt * 16 + r] = m_run[rt];
            l_s[wave][rt * 16 + r] = l;
        }
    }
    __syncthreads();
    float own[RT][4];  // this wave's factor for the accumulator rows g*4+i of tile rt
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = rt * 16 + g * 4 + i;
            float m_all = m_s[0][row];
#pragma unroll
            for (int w = 1; w < kScoredWaves; ++w) m_all = fmaxf(m_all, m_s[w][row]);
            if (a.shape.sinks && row < n_rows && a.n_splits == 1)
                m_all = fmaxf(m_all, a.shape.sinks[kv_head * group + row % group] * kLog2e);
            const float mine = m_s[wave][row];
            own[rt][i] = (mine == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mine - m_all);
        }
    }
    for (int w = 0; w < kScoredWaves; ++w) {
        if (wave == w) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int dt = 0; dt < ND; ++dt) {
                        float* cell = &o_s[rt * 16 + g * 4 + i][dt * 16 + r];
                        const float mine = o[rt][dt][i] * own[rt][i];
                        *cell = (w == 0) ? mine : *cell + mine;
                    }
        }
        __syncthreads();
    }
    if (a.n_splits > 1) {
        // this share's (max, sum, accumulator) of every row, for the merge
        const size_t unit = (static_cast<size_t>(tile) * a.kv_heads + kv_head) * a.n_splits + split;
        float* po = a.part_o + unit * ROWS * DV;
        float* pml = a.part_ml + unit * ROWS * 2;
        for (int row = wave; row < n_rows; row += kScoredWaves) {
            float m_all = m_s[0][row];
#pragma unroll
            for (int w = 1; w < kScoredWaves; ++w) m_all = fmaxf(m_all, m_s[w][row]);
            float sum = 0.f;
#pragma unroll
            for (int w = 0; w < kScoredWaves; ++w) {
                const float mine = m_s[w][row];
                sum += (mine == -INFINITY) ? 0.f : l_s[w][row] * __builtin_amdgcn_exp2f(mine - m_all);
            }
            if (lane == 0) {
                pml[row * 2] = m_all;
                pml[row * 2 + 1] = sum;
            }
            for (int d = lane; d < DV; d += kWave) po[static_cast<size_t>(row) * DV + d] = o_s[row][d];
        }
        return;
    }
    for (int row = wave; row < n_rows; row += kScoredWaves) {
        const int tok = row / group;
        const int head = kv_head * group + (row - tok * group);
        float m_all = m_s[0][row];
#pragma unroll
        for (int w = 1; w < kScoredWaves; ++w) m_all = fmaxf(m_all, m_s[w][row]);
        float den = 0.f;
        if (a.shape.sinks) {
            const float sink = a.shape.sinks[head] * kLog2e;
            m_all = fmaxf(m_all, sink);
            den = __builtin_amdgcn_exp2f(sink - m_all);
        }
#pragma unroll
        for (int w = 0; w < kScoredWaves; ++w) {
            const float mine = m_s[w][row];
            den += (mine == -INFINITY) ? 0.f : l_s[w][row] * __builtin_amdgcn_exp2f(mine - m_all);
        }
        float factor = 1.0f / den;
        if (a.gate) {
            const float z = to_float(a.gate[static_cast<size_t>(first_row_token + tok) * a.gate_stride + head]);
            factor *= 1.0f / (1.0f + __expf(-z));
        }
        bf16_t* dst = a.out + (static_cast<size_t>(first_row_token + tok) * a.q_heads + head) * DV;
        for (int d = lane; d < DV; d += kWave) dst[d] = from_float<bf16_t>(o_s[row][d] * factor);
    }
}

// Joins the shares of a tile's keys: one wave per row (four rows a workgroup).  Lane s fetches the statistics of share
// s (and s + 64, ...), so the common reference and every share's factor are known after one round of loads; the shares'
// sums are then fetched without waiting on one another.
constexpr int kMergeShares = 64;  // shares whose factors one pass keeps in a lane each

__global__ void __launch_bounds__(256) scored_attention_merge_kernel(ScoredArgs a, int rows_per_tile, int DV) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int tile = blockIdx.x;
    const int kv_head = blockIdx.y;
    const int group = a.q_heads / a.kv_heads;
    const int seq = a.tile_seq ? a.tile_seq[tile] : tile;
    const int q0 = a.tile_seq ? a.tile_q0[tile] : 0;
    const int n_tok = min(a.tokens_per_tile, a.seq_q_len[seq] - q0);
    const int n_rows = n_tok * group;
    const int row = blockIdx.z * 4 + wave;
    if (row >= n_rows) return;
    const int first_row_token = a.q_start_loc[seq] + q0;
    const size_t unit0 = (static_cast<size_t>(tile) * a.kv_heads + kv_head) * a.n_splits;
    const int tok = row / group;
    const int head = kv_head * group + (row - tok * group);
    float m_all = -INFINITY;
    for (int sp = lane; sp < a.n_splits; sp += kWave)
        m_all = fmaxf(m_all, a.part_ml[((unit0 + sp) * rows_per_tile + row) * 2]);
    m_all = wave_max(m_all);
    float sink_term = 0.f;  // the sink's share of the denominator, counted once
    if (a.shape.sinks) {
        const float sink = a.shape.sinks[head] * kLog2e;
        m_all = fmaxf(m_all, sink);
        sink_term = __builtin_amdgcn_exp2f(sink - m_all);
    }
    float den = 0.f;        // this lane's shares of it
    float acc[4] = {0.f, 0.f, 0.f, 0.f};  // DV <= 256: four numbers a lane
    for (int base = 0; base < a.n_splits; base += kMergeShares) {
        float mine = 0.f;  // the factor of share base + lane; 0 for a share without keys
        if (base + lane < a.n_splits) {
            const float* ml = a.part_ml + ((unit0 + base + lane) * rows_per_tile + row) * 2;
            mine = (ml[0] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(ml[0] - m_all);
            den += ml[1] * mine;
        }
        const int count = min(kMergeShares, a.n_splits - base);
        for (int sp = 0; sp < count; ++sp) {
            const float f = __shfl(mine, sp, kWave);
            const float* po = a.part_o + ((unit0 + base + sp) * rows_per_tile + row) * DV;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (lane + i * kWave < DV) acc[i] = fmaf(f == 0.f ? 0.f : po[lane + i * kWave], f, acc[i]);
        }
    }
    float factor = 1.0f / (wave_sum(den) + sink_term);
    if (a.gate) {
        const float z = to_float(a.gate[static_cast<size_t>(first_row_token + tok) * a.gate_stride + head]);
        factor *= 1.0f / (1.0f + __expf(-z));
    }
    bf16_t* dst = a.out + (static_cast<size_t>(first_row_token + tok) * a.q_heads + head) * DV;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (lane + i * kWave < DV) dst[lane + i * kWave] = from_float<bf16_t>(acc[i] * factor);
}

template <int D, int DV>
int launch_scored(hipStream_t s, const ScoredArgs& a, int row_tiles) {
    dim3 grid(a.n_tiles, a.kv_heads, a.n_splits);
    if (row_tiles == 1)
        scored_attention_mfma_kernel<D, DV, 1><<<grid, 64 * kScoredWaves, 0, s>>>(a);
    else if (row_tiles == 2)
        scored_attention_mfma_kernel<D, DV, 2><<<grid, 64 * kScoredWaves, 0, s>>>(a);
    else if (row_tiles == 4)
        scored_attention_mfma_kernel<D, DV, 4><<<grid, 64 * kScoredWaves, 0, s>>>(a);
    else
        return CIE_BAD_ARGUMENT;
    if (hipGetLastError() != hipSuccess) return CIE_LAUNCH_FAILED;
    if (a.n_splits > 1)
        scored_attention_merge_kernel<<<dim3(a.n_tiles, a.kv_heads, 4 * row_tiles), 256, 0, s>>>(a, 16 * row_tiles, DV);
    return cie_after_launch();
}

}  // namespace

CIE_API int cie_heads_prepare(void* stream, int dtype, const void* proj, int proj_stride, int q_off, int k_off,
                              int v_off, const float* q_weight, const float* k_weight, int norm_mode, float eps,
                              float temp_coef, int temp_every, const int* positions, const int* seq_of_token,
                              const int* seq_slot, const int* block_table, int table_width, void* q_out,
                              void* k_pool, void* v_pool, int tokens, int q_heads, int kv_heads, int dim, int vdim,
                              int D, int DV, int page_size, int write_kv, const float* cos_table,
                              const float* sin_table, int rot, int neighbours) {
    if (rot < 0 || rot % 2 || rot > dim || (rot > 0 && (!cos_table || !sin_table))) return CIE_BAD_ARGUMENT;
    if (tokens < 0 || q_heads <= 0 || kv_heads <= 0 || dim <= 0 || vdim <= 0 || D < dim || DV < vdim ||
        page_size <= 0 || (page_size & (page_size - 1)) || table_width <= 0 || norm_mode < 0 || norm_mode > 3 ||
        (norm_mode >= 2 && (!q_weight || (write_kv && !k_weight))) || (norm_mode != 0 && !(eps > 0.f)) || temp_every < 0 ||
        q_off < 0 || k_off < 0 || v_off < 0 || proj_stride <= 0)
        return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    int page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
    const long units = static_cast<long>(tokens) * (q_heads + 2 * kv_heads);
    const long blocks = (units + 3) / 4;
    if (blocks > 0x7fffffffL) return CIE_BAD_ARGUMENT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == CIE_F32)
        heads_prepare_kernel<float><<<static_cast<unsigned>(blocks), 256, 0, s>>>(
            static_cast<const float*>(proj), proj_stride, q_off, k_off, v_off, q_weight, k_weight, norm_mode, eps,
            temp_coef, temp_every, positions, seq_of_token, seq_slot, block_table, table_width,
            static_cast<float*>(q_out), static_cast<float*>(k_pool), static_cast<float*>(v_pool), tokens, q_heads,
            kv_heads, dim, vdim, D, DV, page_shift, write_kv, cos_table, sin_table, rot, neighbours);
    else if (dtype == CIE_BF16)
        heads_prepare_kernel<bf16_t><<<static_cast<unsigned>(blocks), 256, 0, s>>>(
            static_cast<const bf16_t*>(proj), proj_stride, q_off, k_off, v_off, q_weight, k_weight, norm_mode, eps,
            temp_coef, temp_every, positions, seq_of_token, seq_slot, block_table, table_width,
            static_cast<bf16_t*>(q_out), static_cast<bf16_t*>(k_pool), static_cast<bf16_t*>(v_pool), tokens, q_heads,
            kv_heads, dim, vdim, D, DV, page_shift, write_kv, cos_table, sin_table, rot, neighbours);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}

CIE_API int cie_scored_attention_generic(void* stream, int dtype, const void* q, const void* k_pool,
                                         const void* v_pool, const int* block_table, int table_width,
                                         const int* positions, const int* seq_of_token, const int* seq_slot,
                                         const void* gate, int gate_stride, void* out, int tokens, int q_heads,
                                         int kv_heads, int D, int DV, int page_size, int window, float scale,
                                         float softcap, const float* slopes, const float* sinks, int chunk,
                                         int keep) {
    if (tokens < 0 || q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads || D <= 0 || D % 8 || DV <= 0 || DV % 8 ||
        D > kWave * kMaxSlices || DV > kWave * kMaxSlices || page_size <= 0 || table_width <= 0 || q_heads > 65535 ||
        (gate && gate_stride < q_heads))
        return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid(tokens, q_heads);
    const size_t lds = (static_cast<size_t>(D) + 4 * DV) * sizeof(float);
    if (chunk < 0 || (chunk > 0 && window > 0) || keep < 0 || (keep > 0 && window <= 0)) return CIE_BAD_ARGUMENT;
    const ScoreShape shape{scale, softcap, slopes, sinks, window, chunk, keep};
    if (dtype == CIE_F32)
        scored_attention_generic_kernel<float><<<grid, 256, lds, s>>>(
            static_cast<const float*>(q), static_cast<const float*>(k_pool), static_cast<const float*>(v_pool),
            block_table, table_width, positions, seq_of_token, seq_slot, static_cast<const float*>(gate), gate_stride,
            static_cast<float*>(out), q_heads, kv_heads, D, DV, page_size, shape);
    else if (dtype == CIE_BF16)
        scored_attention_generic_kernel<bf16_t><<<grid, 256, lds, s>>>(
            static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_pool), static_cast<const bf16_t*>(v_pool),
            block_table, table_width, positions, seq_of_token, seq_slot, static_cast<const bf16_t*>(gate), gate_stride,
            static_cast<bf16_t*>(out), q_heads, kv_heads, D, DV, page_size, shape);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}

// bfloat16 on the matrix cores: (D, DV) one of (64, 64), (128, 128), (64, 128), (128, 64); pages of at least 4 keys;
// a token's heads of one key head fill at most `row_tiles` tiles of 16 rows.
CIE_API int cie_scored_attention_mfma(void* stream, const void* q, const void* k_pool, const void* v_pool,
                                      const int* block_table, int table_width, const int* tile_seq,
                                      const int* tile_q0, int n_tiles, const int* seq_slot, const int* seq_start,
                                      const int* seq_q_len, const int* q_start_loc, const void* gate,
                                      int gate_stride, void* out, int q_heads, int kv_heads, int D, int DV,
                                      int page_size, int tokens_per_tile, int row_tiles, int window, float scale,
                                      float softcap, const float* slopes, const float* sinks, int n_splits,
                                      int keys_per_split, float* part_o, float* part_ml, int chunk, int keep) {
    if (chunk < 0 || (chunk > 0 && window > 0) || keep < 0 || (keep > 0 && window <= 0)) return CIE_BAD_ARGUMENT;
    if (n_tiles < 0 || q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads || page_size < 4 ||
        (page_size & (page_size - 1)) || table_width <= 0 || tokens_per_tile < 1 || kv_heads > 65535 ||
        (tile_seq == nullptr) != (tile_q0 == nullptr) || (gate && gate_stride < q_heads))
        return CIE_BAD_ARGUMENT;
    if (tokens_per_tile * (q_heads / kv_heads) > 16 * row_tiles) return CIE_BAD_ARGUMENT;
    if (n_splits < 1 || n_splits > 65535 ||
        (n_splits > 1 && (keys_per_split < 128 || keys_per_split % 128 || !part_o || !part_ml || DV > 256)))
        return CIE_BAD_ARGUMENT;
    if (n_tiles == 0) return CIE_OK;
    ScoredArgs a;
    a.n_splits = n_splits;
    a.keys_per_split = keys_per_split;
    a.part_o = part_o;
    a.part_ml = part_ml;
    a.q = static_cast<const bf16_t*>(q);
    a.k_pool = static_cast<const bf16_t*>(k_pool);
    a.v_pool = static_cast<const bf16_t*>(v_pool);
    a.block_table = block_table;
    a.table_width = table_width;
    a.tile_seq = tile_seq;
    a.tile_q0 = tile_q0;
    a.seq_slot = seq_slot;
    a.seq_start = seq_start;
    a.seq_q_len = seq_q_len;
    a.q_start_loc = q_start_loc;
    a.gate = static_cast<const bf16_t*>(gate);
    a.gate_stride = gate_stride;
    a.out = static_cast<bf16_t*>(out);
    a.q_heads = q_heads;
    a.kv_heads = kv_heads;
    a.page_shift = 0;
    while ((1 << a.page_shift) < page_size) ++a.page_shift;
    a.tokens_per_tile = tokens_per_tile;
    a.n_tiles = n_tiles;
    a.shape = ScoreShape{scale, softcap, slopes, sinks, window, chunk, keep};
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (D == 64 && DV == 64) return launch_scored<64, 64>(s, a, row_tiles);
    if (D == 128 && DV == 128) return launch_scored<128, 128>(s, a, row_tiles);
    if (D == 64 && DV == 128) return launch_scored<64, 128>(s, a, row_tiles);
    if (D == 128 && DV == 64) return launch_scored<128, 64>(s, a, row_tiles);
    return CIE_BAD_ARGUMENT;
}
