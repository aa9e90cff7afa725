// A memory of outer products per head, S [rows, cols] in float32, that every token fades, adds to and reads:
//
//     S_t[n, p] = decay_t[n] * S_(t-1)[n, p] + in_t[n] * val_t[p]
//
// read after the update (a state-space layer:  y_t[p] = sum_n out_t[n] S_t[n, p] + skip * val_t[p],  decay one number
// per head and token, in/out shared by the heads of a group, val_t scaled by the token's step size for the update),
// or before it, with a bonus on the token's own outer product (time mixing with a decay per row:
// y_t[p] = sum_n out_t[n] (S_(t-1)[n, p] + bonus[n] in_t[n] val_t[p])).  Which of the two, the strides and which
// operands exist are arguments, so that one walk serves both layers; all operands are float32 rows made by the
// kernels in front of it.  The state lives in rows of a state tensor, one per request slot; a step reads what its
// earlier steps left, runs its tokens in order and writes it back, so a sequence may be cut into steps anywhere.
//
// Beside the walk: the step sizes and decays of a state-space layer, the mixes of a token with the one before it
// and the decays of a time-mixing layer, and the norm in groups over a walk's read-out with its gate.
#include "common.h"

namespace {

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float silu_f(float x) { return x * sigmoid_f(x); }
__device__ __forceinline__ float softplus_f(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

struct WalkArgs {
    const float* decay;   // a decay per row: decay[t * ld_decay + head * rows + n]; one per head: decay[t * ld_decay + head]
    long ld_decay;
    const float* in;      // in[t * ld_in + (head / heads_per_group) * rows + n]
    long ld_in;
    const float* out;     // out[t * ld_out + (head / heads_per_group) * rows + n]
    long ld_out;
    int heads_per_group;
    const float* bonus;   // [heads, rows] or null; with the read-out in front of the update only
    const float* val;     // val[t * ld_val + head * cols + p]
    long ld_val;
    const float* val_scale;  // val_scale[t * ld_scale + head] or null: the update takes val * scale
    long ld_scale;
    const float* skip;    // [heads] or null: y += skip[head] * val
    float* state;         // [slots, heads, rows, cols]
    const int* seq_slot;
    const int* q_start_loc;
    float* y;             // [tokens, heads * cols]
    int heads, rows, cols, slice, row_groups, chunk;
};

// One workgroup per (sequence, head, slice of columns).  Thread (column, row group g) keeps rows g * NS .. + NS - 1
// of its column in registers.  Tokens go in chunks: the chunk's row operands are staged in LDS (a row group's numbers
// NS + 4 floats apart from the next group's, so that the groups of a wave read different banks, and every group's
// numbers start at a multiple of 16 bytes: a thread reads them four at a time), every thread walks the chunk's tokens
// in order, the next token's operands on their way from LDS while this token's are worked on, and the row groups'
// shares of y meet in LDS behind the chunk.  The order of every sum depends on the sizes alone, never on what else
// the step holds.  TIME: a decay per row, the read-out in front of the update, a bonus; else one decay per head and
// token, the read-out behind the update.
constexpr int kWalkAhead = 8;         // numbers of each row operand of a chunk that a thread fetches ahead
constexpr int kWalkAheadValues = 4;   // ... and values

// AHEAD: the next chunk's operands are fetched into registers while this chunk is walked (sequences that bring many
// tokens); without it a chunk is staged straight from memory (steps of single tokens, where fetching ahead only costs).
template <int NS, bool TIME, bool AHEAD>
__global__ void __launch_bounds__(512) memory_walk_kernel(WalkArgs a) {
    extern __shared__ float4 lds4[];
    float* lds = reinterpret_cast<float*>(lds4);
    constexpr int Q = NS / 4;
    const int seq = blockIdx.x;
    const int head = blockIdx.y;
    const int col0 = blockIdx.z * a.slice;
    const int RG = a.row_groups;
    const int pitch = NS + 4;
    const int per_token = RG * pitch;
    const int chunk4 = (a.chunk + 3) & ~3;
    float* in_s = lds;                                   // [chunk][RG][pitch]
    float* out_s = in_s + a.chunk * per_token;           // [chunk][RG][pitch]
    float* dec_s = out_s + a.chunk * per_token;          // TIME: [chunk][RG][pitch]; else [chunk]
    float* bon_s = dec_s + (TIME ? a.chunk * per_token : chunk4);  // TIME: [chunk][RG][pitch]
    float* val_s = bon_s + (TIME ? a.chunk * per_token : 0);       // [chunk][slice]
    float* scl_s = val_s + a.chunk * a.slice;            // [chunk]
    float* part_s = scl_s + chunk4;                      // [chunk][RG][slice]

    const int col = threadIdx.x % a.slice;
    const int rg = threadIdx.x / a.slice;
    const bool live = rg < RG && col0 + col < a.cols;
    const int first = a.q_start_loc[seq];
    const int count = a.q_start_loc[seq + 1] - first;
    const int group = head / a.heads_per_group;
    float* mine = a.state + ((static_cast<size_t>(a.seq_slot[seq]) * a.heads + head) * a.rows) * a.cols + col0 + col;
    float S[NS];
#pragma unroll
    for (int i = 0; i < NS; ++i) {
        const int n = rg * NS + i;
        S[i] = (live && n < a.rows) ? mine[static_cast<size_t>(n) * a.cols] : 0.f;
    }
    const float skip = a.skip ? a.skip[head] : 0.f;
    // A chunk's operands are fetched into registers a chunk ahead, so that their way from memory is hidden behind
    // the walk over the chunk before.  Every load stands in straight-line code without a condition (an index past the
    // chunk's last number reads the last one again, a row past the memory's last its last row): behind a load under a
    // condition the compiler waits for it before it issues the next.
    float f_in[kWalkAhead], f_out[kWalkAhead], f_dec[TIME ? kWalkAhead : 1], f_val[kWalkAheadValues];
    float f_scl = 1.f, f_one = 0.f;
    const int padded_rows = RG * NS;
    // which token of a chunk and which row each of the thread's numbers is, and its place in LDS: the same in every chunk
    int slot_t[kWalkAhead], slot_n[kWalkAhead], slot_at[kWalkAhead], value_t[kWalkAheadValues], value_c[kWalkAheadValues];
#pragma unroll
    for (int i = 0; AHEAD && i < kWalkAhead; ++i) {
        const int idx = threadIdx.x + i * blockDim.x;
        slot_t[i] = idx / padded_rows;
        slot_n[i] = idx - slot_t[i] * padded_rows;
        slot_at[i] = slot_t[i] * per_token + (slot_n[i] / NS) * pitch + slot_n[i] % NS;
    }
#pragma unroll
    for (int i = 0; AHEAD && i < kWalkAheadValues; ++i) {
        const int idx = threadIdx.x + i * blockDim.x;
        value_t[i] = idx / a.slice;
        value_c[i] = idx - value_t[i] * a.slice;
    }
#define CIE_WALK_FETCH(from_token)                                                                                    \
    {                                                                                                                 \
        const int fetch_n = min(a.chunk, count - (from_token));                                                       \
        _Pragma("unroll") for (int i = 0; i < kWalkAhead; ++i) {                                                      \
            const int n = min(slot_n[i], a.rows - 1);                                                                 \
            const size_t token = static_cast<size_t>(first + (from_token) + min(slot_t[i], fetch_n - 1));             \
            f_in[i] = a.in[token * a.ld_in + group * a.rows + n];                                                     \
            f_out[i] = a.out[token * a.ld_out + group * a.rows + n];                                                  \
            if (TIME) f_dec[i] = a.decay[token * a.ld_decay + head * a.rows + n];                                     \
        }                                                                                                             \
        _Pragma("unroll") for (int i = 0; i < kWalkAheadValues; ++i) {                                                \
            const int c = min(col0 + value_c[i], a.cols - 1);                                                         \
            f_val[i] = a.val[static_cast<size_t>(first + (from_token) + min(value_t[i], fetch_n - 1)) * a.ld_val +    \
                             head * a.cols + c];                                                                      \
        }                                                                                                             \
        {                                                                                                             \
            const size_t token = static_cast<size_t>(first + (from_token) + min(static_cast<int>(threadIdx.x), fetch_n - 1)); \
            if (a.val_scale) f_scl = a.val_scale[token * a.ld_scale + head];                                          \
            if (!TIME) f_one = a.decay[token * a.ld_decay + head];                                                    \
        }                                                                                                             \
    }
    if (AHEAD && count > 0) CIE_WALK_FETCH(0)
    for (int from = 0; from < count; from += a.chunk) {
        const int n_tok = min(a.chunk, count - from);
        __syncthreads();  // (the chunk before has been summed)
        if (!AHEAD) {
            for (int idx = threadIdx.x; idx < n_tok * padded_rows; idx += blockDim.x) {
                const int t = idx / padded_rows;
                const int n = idx - t * padded_rows;
                const int at = t * per_token + (n / NS) * pitch + n % NS;
                const size_t token = static_cast<size_t>(first + from + t);
                const bool real = n < a.rows;
                const float x = real ? a.in[token * a.ld_in + group * a.rows + n] : 0.f;
                in_s[at] = x;
                out_s[at] = real ? a.out[token * a.ld_out + group * a.rows + n] : 0.f;
                if (TIME) {
                    dec_s[at] = real ? a.decay[token * a.ld_decay + head * a.rows + n] : 0.f;
                    bon_s[at] = (real && a.bonus) ? a.bonus[head * a.rows + n] * x : 0.f;
                }
            }
            for (int idx = threadIdx.x; idx < n_tok * a.slice; idx += blockDim.x) {
                const int t = idx / a.slice;
                const int c = idx - t * a.slice;
                const size_t token = static_cast<size_t>(first + from + t);
                val_s[idx] = col0 + c < a.cols ? a.val[token * a.ld_val + head * a.cols + col0 + c] : 0.f;
            }
            for (int t = threadIdx.x; t < n_tok; t += blockDim.x) {
                const size_t token = static_cast<size_t>(first + from + t);
                scl_s[t] = a.val_scale ? a.val_scale[token * a.ld_scale + head] : 1.f;
                if (!TIME) dec_s[t] = a.decay[token * a.ld_decay + head];
            }
        }
#pragma unroll
        for (int i = 0; AHEAD && i < kWalkAhead; ++i) {
            if (slot_t[i] < n_tok) {
                const int n = slot_n[i];
                const int at = slot_at[i];
                const bool real = n < a.rows;
                in_s[at] = real ? f_in[i] : 0.f;
                out_s[at] = real ? f_out[i] : 0.f;
                if (TIME) {
                    dec_s[at] = real ? f_dec[i] : 0.f;
                    bon_s[at] = (real && a.bonus) ? a.bonus[head * a.rows + n] * f_in[i] : 0.f;
                }
            }
        }
#pragma unroll
        for (int i = 0; AHEAD && i < kWalkAheadValues; ++i) {
            if (value_t[i] < n_tok) val_s[value_t[i] * a.slice + value_c[i]] = col0 + value_c[i] < a.cols ? f_val[i] : 0.f;
        }
        if (AHEAD && static_cast<int>(threadIdx.x) < n_tok) {
            scl_s[threadIdx.x] = f_scl;
            if (!TIME) dec_s[threadIdx.x] = f_one;
        }
        __syncthreads();
        if (AHEAD && from + a.chunk < count) CIE_WALK_FETCH(from + a.chunk)
        if (rg < RG) {
            const int base = rg * pitch;
            float4 in_next[Q], out_next[Q], dec_next[TIME ? Q : 1], bon_next[TIME ? Q : 1];
            // (a token's value and its scale are multiplied when the token's turn comes, not behind their loads: the
            // product there would make the wave wait for LDS at the head of every token)
            float v_next = val_s[col], s_next = scl_s[0];
            float d_next = TIME ? 0.f : dec_s[0];
#pragma unroll
            for (int r = 0; r < Q; ++r) {
                in_next[r] = reinterpret_cast<const float4*>(in_s + base)[r];
                out_next[r] = reinterpret_cast<const float4*>(out_s + base)[r];
                if (TIME) {
                    dec_next[r] = reinterpret_cast<const float4*>(dec_s + base)[r];
                    bon_next[r] = reinterpret_cast<const float4*>(bon_s + base)[r];
                }
            }
            for (int t = 0; t < n_tok; ++t) {
                float4 in_now[Q], out_now[Q], dec_now[TIME ? Q : 1], bon_now[TIME ? Q : 1];
                const float v = v_next * s_next;
                const float d = d_next;
#pragma unroll
                for (int r = 0; r < Q; ++r) {
                    in_now[r] = in_next[r];
                    out_now[r] = out_next[r];
                    if (TIME) {
                        dec_now[r] = dec_next[r];
                        bon_now[r] = bon_next[r];
                    }
                }
                const int ahead = min(t + 1, n_tok - 1);  // (the last token is read twice: no condition around the reads)
                const int at = ahead * per_token + base;
                v_next = val_s[ahead * a.slice + col];
                s_next = scl_s[ahead];
                if (!TIME) d_next = dec_s[ahead];
#pragma unroll
                for (int r = 0; r < Q; ++r) {
                    in_next[r] = reinterpret_cast<const float4*>(in_s + at)[r];
                    out_next[r] = reinterpret_cast<const float4*>(out_s + at)[r];
                    if (TIME) {
                        dec_next[r] = reinterpret_cast<const float4*>(dec_s + at)[r];
                        bon_next[r] = reinterpret_cast<const float4*>(bon_s + at)[r];
                    }
                }
                float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
                for (int r = 0; r < Q; ++r) {
                    const float4 k4 = in_now[r], q4 = out_now[r];
                    if (TIME) {
                        const float4 w4 = dec_now[r], b4 = bon_now[r];
                        a0 = fmaf(q4.x, fmaf(b4.x, v, S[4 * r + 0]), a0);
                        a1 = fmaf(q4.y, fmaf(b4.y, v, S[4 * r + 1]), a1);
                        a2 = fmaf(q4.z, fmaf(b4.z, v, S[4 * r + 2]), a2);
                        a3 = fmaf(q4.w, fmaf(b4.w, v, S[4 * r + 3]), a3);
                        S[4 * r + 0] = fmaf(w4.x, S[4 * r + 0], k4.x * v);
                        S[4 * r + 1] = fmaf(w4.y, S[4 * r + 1], k4.y * v);
                        S[4 * r + 2] = fmaf(w4.z, S[4 * r + 2], k4.z * v);
                        S[4 * r + 3] = fmaf(w4.w, S[4 * r + 3], k4.w * v);
                    } else {
                        S[4 * r + 0] = fmaf(d, S[4 * r + 0], k4.x * v);
                        S[4 * r + 1] = fmaf(d, S[4 * r + 1], k4.y * v);
                        S[4 * r + 2] = fmaf(d, S[4 * r + 2], k4.z * v);
                        S[4 * r + 3] = fmaf(d, S[4 * r + 3], k4.w * v);
                        a0 = fmaf(q4.x, S[4 * r + 0], a0);
                        a1 = fmaf(q4.y, S[4 * r + 1], a1);
                        a2 = fmaf(q4.z, S[4 * r + 2], a2);
                        a3 = fmaf(q4.w, S[4 * r + 3], a3);
                    }
                }
                part_s[(t * RG + rg) * a.slice + col] = (a0 + a1) + (a2 + a3);
            }
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < n_tok * a.slice; idx += blockDim.x) {
            const int t = idx / a.slice;
            const int c = idx - t * a.slice;
            if (col0 + c >= a.cols) continue;
            float sum = 0.f;
            for (int g = 0; g < RG; ++g) sum += part_s[(t * RG + g) * a.slice + c];
            sum = fmaf(skip, val_s[idx], sum);
            a.y[static_cast<size_t>(first + from + t) * a.heads * a.cols + head * a.cols + col0 + c] = sum;
        }
    }
    if (!live) return;
#pragma unroll
    for (int i = 0; i < NS; ++i) {
        const int n = rg * NS + i;
        if (n < a.rows) mine[static_cast<size_t>(n) * a.cols] = S[i];
    }
}
#undef CIE_WALK_FETCH

// ---------------------------------------------------------------------------------------------- the walk in blocks
// The first form of the walk (one decay per head and token, the read-out behind the update) for sequences that
// bring many tokens: blocks of 32 tokens on the matrix cores, float32 throughout (`v_mfma_f32_16x16x4_f32`), and only
// what has to wait for the block before it waits.  With S the memory in front of a block of n tokens, i and j tokens
// of the block, L_i the sum of the logarithms of the decays of the block's tokens 0 .. i, and w_j = val_j * scale_j:
//     y_i   = exp(L_i) * (S^T out_i)  +  sum_{j <= i} exp(L_i - L_j) (out_i . in_j) w_j   (+ skip * val_i)
//     S_new = exp(L_(n-1)) * S  +  sum_j exp(L_(n-1) - L_j) in_j w_j^T
// (every exponent is at most zero).  Three kernels, as for the memory with a fixed decay in recurrent.hip:
// `walk_block_sums_kernel`, every block at once, makes the second term of y and of S_new (into the block's place of
// `sums`) and the block's whole decay; `walk_scan_kernel`, one thread per number of the memory, goes over a
// sequence's blocks in order: the block's place gets the S in front of it, and S moves on; `walk_block_reads_kernel`,
// every block at once, adds the first term of y.  Block b of sequence s has place first_token(s) / 32 + s + b.  Rows
// are padded to whole tiles of 16 (`padded`), a workgroup takes up to 128 columns (a panel) rounded up to tiles of
// 16 (`cols16` columns a row of `sums`).  Operand layouts of the 16 x 16 x 4 product: lane (l16 = lane % 16,
// g = lane / 16) gives A[l16][g] and B[g][l16] and gets rows 4 g .. 4 g + 3 of column l16; which four numbers of a
// sum a product takes does not matter as long as both operands agree, so a lane reads four neighbouring numbers at
// once and spends them on four products.
typedef float acc4_t __attribute__((ext_vector_type(4)));
constexpr int kBlockTokens = 32;
constexpr int kPanelCols = 128;
constexpr int kScoreStride = kBlockTokens + 4;

// rows of a panel of values in LDS start 16 banks apart: the four tokens that a product reads then touch every bank
__host__ __device__ inline int panel_stride(int cols) { return cols % 32 == 0 ? cols + 16 : cols; }

struct BlockArgs {
    const float* log_decay;  // log_decay[t * ld_decay + head]
    long ld_decay;
    const float* in;         // in[t * ld_in + (head / heads_per_group) * rows + n]
    long ld_in;
    const float* out;
    long ld_out;
    int heads_per_group;
    const float* val;        // val[t * ld_val + head * cols + p]
    long ld_val;
    const float* val_scale;  // val_scale[t * ld_scale + head] or null
    long ld_scale;
    const float* skip;       // [heads] or null
    float* state;            // [slots, heads, rows, cols]
    const int* seq_slot;
    const int* q_start_loc;
    float* y;                // [tokens, heads * cols]
    float* sums;             // [places, heads, padded, cols16]
    float* totals;           // [places, heads]: exp of the block's summed log decays
    int heads, rows, cols, padded, cols16;
};

// L_0 .. L_31 of a block into `cum` (tokens past the block's last repeat its L), by one thread
__device__ __forceinline__ void block_logs(float* cum, const BlockArgs& a, int first_token, int cn, int head) {
    if (threadIdx.x == 0) {
        float sum = 0.f;
        for (int t = 0; t < kBlockTokens; ++t) {
            if (t < cn) sum += a.log_decay[static_cast<size_t>(first_token + t) * a.ld_decay + head];
            cum[t] = sum;
        }
    }
}

// a block's rows of `src` (in or out) into LDS rows of `stride` floats; rows past the memory's last and tokens past
// the block's last are zero
__device__ __forceinline__ void stage_block_rows(float* dst, int stride, const float* __restrict__ src, long ld,
                                                 int first_token, int cn, int offset, int rows, int padded) {
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    for (int t = wave; t < kBlockTokens; t += 4) {
        const float* row = src + static_cast<size_t>(first_token + min(t, cn - 1)) * ld + offset;
        for (int n = lane; n < padded; n += kWave) dst[t * stride + n] = (t < cn && n < rows) ? row[n] : 0.f;
    }
}

__global__ void __launch_bounds__(256) walk_block_sums_kernel(BlockArgs a) {
    const int seq = blockIdx.x / a.heads;
    const int head = blockIdx.x - seq * a.heads;
    const int first = a.q_start_loc[seq];
    const int count = a.q_start_loc[seq + 1] - first;
    const int c0 = blockIdx.y * kBlockTokens;
    if (c0 >= count) return;                             // (the whole workgroup: the grid is sized for the longest sequence)
    const int cn = min(kBlockTokens, count - c0);
    const int panel0 = blockIdx.z * kPanelCols;
    const int cols = min(kPanelCols, a.cols16 - panel0);
    const int col_tiles = cols / 16;
    const int padded = a.padded;
    const int stride = padded + 4;
    const int vstride = panel_stride(cols);
    extern __shared__ float4 lds4[];
    float* q_s = reinterpret_cast<float*>(lds4);          // [32][stride]: the read-out's rows
    float* k_s = q_s + kBlockTokens * stride;            // [32][stride]: the update's rows
    float* v_s = k_s + kBlockTokens * stride;            // [32][vstride]: the scaled values
    float* p_s = v_s + kBlockTokens * vstride;           // [32][36]: exp(L_i - L_j) (out_i . in_j), zero above the diagonal
    float* cum = p_s + kBlockTokens * kScoreStride;      // [32]
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int l16 = lane % 16;
    const int g = lane / 16;
    const int tiles = padded / 16;
    const int offset = (head / a.heads_per_group) * a.rows;
    block_logs(cum, a, first + c0, cn, head);
    stage_block_rows(q_s, stride, a.out, a.ld_out, first + c0, cn, offset, a.rows, padded);
    stage_block_rows(k_s, stride, a.in, a.ld_in, first + c0, cn, offset, a.rows, padded);
    for (int t = wave; t < kBlockTokens; t += 4) {
        const size_t token = static_cast<size_t>(first + c0 + min(t, cn - 1));
        const float scale = a.val_scale ? a.val_scale[token * a.ld_scale + head] : 1.f;
        const float* src = a.val + token * a.ld_val + head * a.cols;
        for (int c = lane; c < cols; c += kWave)
            v_s[t * vstride + c] = (t < cn && panel0 + c < a.cols) ? src[panel0 + c] * scale : 0.f;
    }
    __syncthreads();
    {   // this wave's tile of the scores (the tile above the diagonal is zero)
        const int ti = wave >> 1, tj = wave & 1;
        acc4_t p = {0.f, 0.f, 0.f, 0.f};
        if (tj <= ti) {
            const float* qa = q_s + (16 * ti + l16) * stride + 4 * g;
            const float* kb = k_s + (16 * tj + l16) * stride + 4 * g;
            acc4_t p1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
            for (int m = 0; m < tiles; ++m) {
                const float4 x = *reinterpret_cast<const float4*>(qa + 16 * m);
                const float4 b = *reinterpret_cast<const float4*>(kb + 16 * m);
                p = __builtin_amdgcn_mfma_f32_16x16x4f32(x.x, b.x, p, 0, 0, 0);
                p1 = __builtin_amdgcn_mfma_f32_16x16x4f32(x.y, b.y, p1, 0, 0, 0);
                p = __builtin_amdgcn_mfma_f32_16x16x4f32(x.z, b.z, p, 0, 0, 0);
                p1 = __builtin_amdgcn_mfma_f32_16x16x4f32(x.w, b.w, p1, 0, 0, 0);
            }
            p += p1;
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int i = 16 * ti + 4 * g + r, j = 16 * tj + l16;
            p_s[i * kScoreStride + j] = i >= j ? p[r] * expf(cum[i] - cum[j]) : 0.f;
        }
    }
    __syncthreads();
    float k_fade[kBlockTokens / 4];
#pragma unroll
    for (int kk = 0; kk < kBlockTokens / 4; ++kk) k_fade[kk] = expf(cum[kBlockTokens - 1] - cum[4 * kk + g]);
    const int place = first / kBlockTokens + seq + blockIdx.y;
    if (threadIdx.x == 0 && blockIdx.z == 0) a.totals[static_cast<size_t>(place) * a.heads + head] = expf(cum[kBlockTokens - 1]);
    float* sum_rows = a.sums + (static_cast<size_t>(place) * a.heads + head) * padded * a.cols16 + panel0;
    const float skip = a.skip ? a.skip[head] : 0.f;
    for (int ct = wave; ct < col_tiles; ct += 4) {       // this wave's tiles of columns
        float vb[kBlockTokens / 4];
#pragma unroll
        for (int kk = 0; kk < kBlockTokens / 4; ++kk) vb[kk] = v_s[(4 * kk + g) * vstride + 16 * ct + l16];
        // the block's own share of y
        acc4_t o0 = {0.f, 0.f, 0.f, 0.f}, o1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < kBlockTokens / 4; ++kk) {
            o0 = __builtin_amdgcn_mfma_f32_16x16x4f32(p_s[l16 * kScoreStride + 4 * kk + g], vb[kk], o0, 0, 0, 0);
            o1 = __builtin_amdgcn_mfma_f32_16x16x4f32(p_s[(16 + l16) * kScoreStride + 4 * kk + g], vb[kk], o1, 0, 0, 0);
        }
        const int col = panel0 + 16 * ct + l16;
        if (col < a.cols) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = 4 * g + r;
                const size_t token = static_cast<size_t>(first + c0);
                float* dst = a.y + token * a.heads * a.cols + head * a.cols + col;
                const float* raw = a.val + token * a.ld_val + head * a.cols + col;
                if (i < cn) dst[static_cast<size_t>(i) * a.heads * a.cols] = fmaf(skip, raw[static_cast<size_t>(i) * a.ld_val], o0[r]);
                if (16 + i < cn)
                    dst[static_cast<size_t>(16 + i) * a.heads * a.cols] = fmaf(skip, raw[static_cast<size_t>(16 + i) * a.ld_val], o1[r]);
            }
        }
        // what the block adds to the memory
        for (int rt = 0; rt < tiles; ++rt) {
            acc4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < kBlockTokens / 4; ++kk)
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(k_s[(4 * kk + g) * stride + 16 * rt + l16] * k_fade[kk], vb[kk],
                                                          acc, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 4; ++r) sum_rows[static_cast<size_t>(16 * rt + 4 * g + r) * a.cols16 + 16 * ct + l16] = acc[r];
        }
    }
}

// One thread per number of a head's memory (rows and columns padded as `sums` has them): over the sequence's blocks in
// order, the block's place gets the memory in front of the block, and the memory moves on by the block's sum.
__global__ void __launch_bounds__(256) walk_scan_kernel(BlockArgs a) {
    const int seq = blockIdx.x / a.heads;
    const int head = blockIdx.x - seq * a.heads;
    const int e = blockIdx.y * blockDim.x + threadIdx.x;
    if (e >= a.padded * a.cols16) return;
    const int first = a.q_start_loc[seq];
    const int count = a.q_start_loc[seq + 1] - first;
    if (count <= 0) return;
    const int row = e / a.cols16;
    const int col = e - row * a.cols16;
    const bool real = row < a.rows && col < a.cols;
    float* mem = a.state + ((static_cast<size_t>(a.seq_slot[seq]) * a.heads + head) * a.rows + row) * a.cols + col;
    float S = real ? *mem : 0.f;
    const int blocks = (count + kBlockTokens - 1) / kBlockTokens;
    const size_t place0 = static_cast<size_t>(first / kBlockTokens + seq);
    const size_t step = static_cast<size_t>(a.heads) * a.padded * a.cols16;
    float* at = a.sums + (place0 * a.heads + head) * a.padded * a.cols16 + e;
    const float* fade = a.totals + place0 * a.heads + head;
    float add = at[0];
    float whole = fade[0];
    for (int b = 0; b < blocks; ++b) {
        const int ahead = min(b + 1, blocks - 1);
        const float next = at[static_cast<size_t>(ahead) * step];  // (asked for before this block's place is written)
        const float next_whole = fade[static_cast<size_t>(ahead) * a.heads];
        at[static_cast<size_t>(b) * step] = S;
        S = fmaf(whole, S, add);
        add = next;
        whole = next_whole;
    }
    if (real) *mem = S;
}

__global__ void __launch_bounds__(256) walk_block_reads_kernel(BlockArgs a) {
    const int seq = blockIdx.x / a.heads;
    const int head = blockIdx.x - seq * a.heads;
    const int first = a.q_start_loc[seq];
    const int count = a.q_start_loc[seq + 1] - first;
    const int c0 = blockIdx.y * kBlockTokens;
    if (c0 >= count) return;
    const int cn = min(kBlockTokens, count - c0);
    const int panel0 = blockIdx.z * kPanelCols;
    const int col_tiles = min(kPanelCols, a.cols16 - panel0) / 16;
    const int padded = a.padded;
    const int stride = padded + 4;
    extern __shared__ float4 lds4[];
    float* q_s = reinterpret_cast<float*>(lds4);          // [32][stride]
    float* cum = q_s + kBlockTokens * stride;            // [32]
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int l16 = lane % 16;
    const int g = lane / 16;
    const int tiles = padded / 16;
    block_logs(cum, a, first + c0, cn, head);
    stage_block_rows(q_s, stride, a.out, a.ld_out, first + c0, cn, (head / a.heads_per_group) * a.rows, a.rows, padded);
    __syncthreads();
    const int place = first / kBlockTokens + seq + blockIdx.y;
    const float* before = a.sums + (static_cast<size_t>(place) * a.heads + head) * padded * a.cols16 + panel0;
    for (int ct = wave; ct < col_tiles; ct += 4) {
        acc4_t o0 = {0.f, 0.f, 0.f, 0.f}, o1 = {0.f, 0.f, 0.f, 0.f};
        const float* rows = before + static_cast<size_t>(4 * g) * a.cols16 + 16 * ct + l16;
#pragma unroll 2
        for (int m = 0; m < tiles; ++m) {
            const float4 a0 = *reinterpret_cast<const float4*>(q_s + l16 * stride + 16 * m + 4 * g);
            const float4 a1 = *reinterpret_cast<const float4*>(q_s + (16 + l16) * stride + 16 * m + 4 * g);
            const float* s = rows + static_cast<size_t>(16 * m) * a.cols16;
            const float b0 = s[0], b1 = s[a.cols16], b2 = s[2 * a.cols16], b3 = s[3 * a.cols16];
            o0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a0.x, b0, o0, 0, 0, 0);
            o1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a1.x, b0, o1, 0, 0, 0);
            o0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a0.y, b1, o0, 0, 0, 0);
            o1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a1.y, b1, o1, 0, 0, 0);
            o0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a0.z, b2, o0, 0, 0, 0);
            o1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a1.z, b2, o1, 0, 0, 0);
            o0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a0.w, b3, o0, 0, 0, 0);
            o1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a1.w, b3, o1, 0, 0, 0);
        }
        const int col = panel0 + 16 * ct + l16;
        if (col < a.cols) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = 4 * g + r;
                float* dst = a.y + static_cast<size_t>(first + c0) * a.heads * a.cols + head * a.cols + col;
                if (i < cn) dst[static_cast<size_t>(i) * a.heads * a.cols] += o0[r] * expf(cum[i]);
                if (16 + i < cn) dst[static_cast<size_t>(16 + i) * a.heads * a.cols] += o1[r] * expf(cum[16 + i]);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------- state-space steps
// Per (token, head): the step size dt = softplus(raw + bias), the decay's logarithm -exp(a_log) * dt and the decay,
// float32.
template <typename T>
__global__ void __launch_bounds__(256)
space_steps_kernel(const T* __restrict__ raw, long ld, const float* __restrict__ bias, const float* __restrict__ a_log,
                   float* __restrict__ steps, float* __restrict__ decay, float* __restrict__ log_decay, long count,
                   int heads) {
    const long idx = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= count) return;
    const long token = idx / heads;
    const int head = static_cast<int>(idx - token * heads);
    const float dt = softplus_f(to_float(raw[token * ld + head]) + bias[head]);
    const float fade = -expf(a_log[head]) * dt;
    steps[idx] = dt;
    log_decay[idx] = fade;
    decay[idx] = expf(fade);
}

// ---------------------------------------------------------------------------------------------- token shift
// mixes[s][t] = h_t + (h_(t-1) - h_t) * mu[s] for each of `n_mix` weight rows mu[s]; the token in front of a step's
// first token comes from the state (zeros for a new sequence).  The state is moved on by `time_decay_kernel`, which
// runs behind everything that reads it.
template <typename T>
__global__ void __launch_bounds__(256)
shift_mix_kernel(const T* __restrict__ h, long ldh, const float* __restrict__ before, const float* __restrict__ mu,
                 const int* __restrict__ seq_of_token, const int* __restrict__ seq_slot,
                 const int* __restrict__ q_start_loc, T* __restrict__ mixes, int tokens, int width, int n_mix) {
    const int token = blockIdx.x;
    const int seq = seq_of_token[token];
    const bool first = token == q_start_loc[seq];
    const T* row = h + static_cast<size_t>(token) * ldh;
    const T* prev = h + static_cast<size_t>(token - 1) * ldh;
    const float* kept = before + static_cast<size_t>(seq_slot[seq]) * width;
    // (blockIdx.y: the token's channels in blocks, so that a single token's row is not one thread's loop of loads)
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < width; c += blockDim.x * gridDim.y) {
        const float x = to_float(row[c]);
        const float d = (first ? kept[c] : to_float(prev[c])) - x;
        for (int s = 0; s < n_mix; ++s)
            mixes[(static_cast<size_t>(s) * tokens + token) * width + c] =
                from_float<T>(fmaf(d, mu[static_cast<size_t>(s) * width + c], x));
    }
}

// w[t, c] = exp(-exp(w2[c, :] . tanh(low[t, :]) + w0[c])): the decay of every key channel from the low-rank
// projection of its mix (float32 [tokens, rank]).  `w2t` is w2 transposed, [rank, channels], so that neighbouring
// threads read neighbouring numbers.  A workgroup per (token, block of channels); tanh(low) is staged in LDS.  Also
// moves the token-shift state on: the step's last token of every sequence leaves its input row there.
template <typename T>
__global__ void __launch_bounds__(256)
time_decay_kernel(const float* __restrict__ low, const T* __restrict__ w2t, const float* __restrict__ w0,
                  float* __restrict__ decay, int channels, int rank, const T* __restrict__ h, long ldh,
                  float* __restrict__ before, const int* __restrict__ seq_of_token, const int* __restrict__ seq_slot,
                  const int* __restrict__ q_start_loc, int width) {
    extern __shared__ float bent[];
    const int token = blockIdx.x;
    for (int r = threadIdx.x; r < rank; r += blockDim.x) bent[r] = tanhf(low[static_cast<size_t>(token) * rank + r]);
    __syncthreads();
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < channels; c += blockDim.x * gridDim.y) {
        float sum = 0.f, sum1 = 0.f;
        int r = 0;
        for (; r + 1 < rank; r += 2) {
            sum = fmaf(to_float(w2t[static_cast<size_t>(r) * channels + c]), bent[r], sum);
            sum1 = fmaf(to_float(w2t[static_cast<size_t>(r + 1) * channels + c]), bent[r + 1], sum1);
        }
        if (r < rank) sum = fmaf(to_float(w2t[static_cast<size_t>(r) * channels + c]), bent[r], sum);
        decay[static_cast<size_t>(token) * channels + c] = expf(-expf((sum + sum1) + w0[c]));
    }
    const int seq = seq_of_token[token];
    if (token + 1 == q_start_loc[seq + 1]) {
        float* kept = before + static_cast<size_t>(seq_slot[seq]) * width;
        const T* row = h + static_cast<size_t>(token) * ldh;
        for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < width; c += blockDim.x * gridDim.y) kept[c] = to_float(row[c]);
    }
}

// ---------------------------------------------------------------------------------------------- read-out norm
// out[t] = norm(y[t] * silu(gate[t])) * weight      (gate_first: the gate comes before the norm)
// out[t] = norm(y[t]) * weight * silu(gate[t])      (otherwise)
// with the norm over `groups` equal consecutive parts of the row, each divided by sqrt(mean(part^2) + eps).  y is
// float32 [tokens, width]; the gate a view of T rows `ldg` apart; everything inside is float32.  One workgroup per
// token, a wave per group in turn, the row staged in LDS.
template <typename T>
__global__ void __launch_bounds__(1024)
gated_group_norm_kernel(const float* __restrict__ y, const T* __restrict__ gate, long ldg,
                        const float* __restrict__ weight, T* __restrict__ out, int width, int groups, float eps,
                        int gate_first) {
    extern __shared__ float staged[];  // [width], then [groups]
    float* inverse = staged + width;
    const size_t token = blockIdx.x;
    const float* row = y + token * width;
    const T* g_row = gate ? gate + token * ldg : nullptr;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        float x = row[c];
        if (g_row && gate_first) x *= silu_f(to_float(g_row[c]));
        staged[c] = x;
    }
    __syncthreads();
    const int lane = threadIdx.x % kWave;
    const int waves = blockDim.x / kWave;
    const int per = width / groups;
    for (int g = threadIdx.x / kWave; g < groups; g += waves) {
        float sum_sq = 0.f;
        for (int c = lane; c < per; c += kWave) {
            const float x = staged[g * per + c];
            sum_sq += x * x;
        }
        sum_sq = wave_sum(sum_sq);
        if (lane == 0) inverse[g] = 1.0f / sqrtf(sum_sq / static_cast<float>(per) + eps);
    }
    __syncthreads();
    T* dst = out + token * width;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        float x = staged[c] * inverse[c / per];
        if (weight) x *= weight[c];
        if (g_row && !gate_first) x *= silu_f(to_float(g_row[c]));
        dst[c] = from_float<T>(x);
    }
}

}  // namespace

// The walk (see the head of this file).  `time_form`: a decay per row ([tokens, heads * rows]), the read-out in front of
// the update, `bonus` if given; else one decay per head and token ([tokens, heads]) and the read-out behind the update.
// `rows_per_thread` in {4, 8, 16, 32, 64}; `row_groups * rows_per_thread >= rows`; `slice` columns a workgroup,
// `slice * row_groups <= 512` threads; `chunk` tokens staged at once; `ahead`: the next chunk's operands are fetched
// into registers while a chunk is walked (for sequences that bring many tokens).
CIE_API int cie_memory_walk(void* stream, const float* decay, long ld_decay, const float* in, long ld_in,
                            const float* out, long ld_out, int heads_per_group, const float* bonus, const float* val,
                            long ld_val, const float* val_scale, long ld_scale, const float* skip, float* state,
                            const int* seq_slot, const int* q_start_loc, float* y, int sequences, int heads, int rows,
                            int cols, int rows_per_thread, int row_groups, int slice, int chunk, int time_form,
                            int ahead) {
    if (sequences < 0 || heads <= 0 || heads > 65535 || rows <= 0 || cols <= 0 || heads_per_group <= 0 ||
        heads % heads_per_group || row_groups <= 0 || slice <= 0 || chunk <= 0 ||
        static_cast<long>(rows_per_thread) * row_groups < rows || slice * row_groups > 512 || !decay || !in || !out ||
        !val || !state || !y || (bonus && !time_form))
        return CIE_BAD_ARGUMENT;
    const int slices = (cols + slice - 1) / slice;
    if (slices > 65535) return CIE_BAD_ARGUMENT;
    const int per_token = row_groups * (rows_per_thread + 4);
    const int chunk4 = (chunk + 3) & ~3;
    const size_t floats = static_cast<size_t>(chunk) * ((time_form ? 4 : 2) * per_token + slice +
                                                        static_cast<size_t>(row_groups) * slice) +
                          (time_form ? 1 : 2) * chunk4;
    if (floats * sizeof(float) > 64 * 1024) return CIE_BAD_ARGUMENT;
    {   // what a thread fetches ahead must hold a chunk
        const int launch = ((slice * row_groups + kWave - 1) / kWave) * kWave;
        if (static_cast<long>(chunk) * row_groups * rows_per_thread > static_cast<long>(kWalkAhead) * launch ||
            static_cast<long>(chunk) * slice > static_cast<long>(kWalkAheadValues) * launch || chunk > launch)
            return CIE_BAD_ARGUMENT;
    }
    if (sequences == 0) return CIE_OK;
    WalkArgs a{decay, ld_decay, in, ld_in, out, ld_out, heads_per_group, bonus, val, ld_val, val_scale, ld_scale,
               skip, state, seq_slot, q_start_loc, y, heads, rows, cols, slice, row_groups, chunk};
    const int threads = ((slice * row_groups + kWave - 1) / kWave) * kWave;
    const dim3 grid(sequences, heads, slices);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t lds = floats * sizeof(float);
#define CIE_WALK(NS)                                                                                \
    if (time_form && ahead) memory_walk_kernel<NS, true, true><<<grid, threads, lds, s>>>(a);           \
    else if (time_form) memory_walk_kernel<NS, true, false><<<grid, threads, lds, s>>>(a);             \
    else if (ahead) memory_walk_kernel<NS, false, true><<<grid, threads, lds, s>>>(a);                 \
    else memory_walk_kernel<NS, false, false><<<grid, threads, lds, s>>>(a)
    if (rows_per_thread == 4) { CIE_WALK(4); }
    else if (rows_per_thread == 8) { CIE_WALK(8); }
    else if (rows_per_thread == 16) { CIE_WALK(16); }
    else if (rows_per_thread == 32) { CIE_WALK(32); }
    else if (rows_per_thread == 64) { CIE_WALK(64); }
    else return CIE_BAD_ARGUMENT;
#undef CIE_WALK
    return cie_after_launch();
}

// The first form of the walk in blocks of 32 tokens on the matrix cores (see above).  `sums` holds
// (tokens / 32 + sequences + 1) * heads * padded * cols16 floats and `totals` (tokens / 32 + sequences + 1) * heads,
// with padded and cols16 the rows and columns rounded up to multiples of 16.
CIE_API int cie_memory_walk_blocks(void* stream, const float* log_decay, long ld_decay, const float* in, long ld_in,
                                   const float* out, long ld_out, int heads_per_group, const float* val, long ld_val,
                                   const float* val_scale, long ld_scale, const float* skip, float* state,
                                   const int* seq_slot, const int* q_start_loc, float* y, float* sums, float* totals,
                                   int tokens, int sequences, int heads, int rows, int cols) {
    if (sequences < 0 || tokens < 0 || heads <= 0 || rows <= 0 || cols <= 0 || heads_per_group <= 0 ||
        heads % heads_per_group || !log_decay || !in || !out || !val || !state || !y || !sums || !totals)
        return CIE_BAD_ARGUMENT;
    const int padded = (rows + 15) / 16 * 16;
    const int cols16 = (cols + 15) / 16 * 16;
    const int panels = (cols16 + kPanelCols - 1) / kPanelCols;
    const int most_blocks = (tokens + kBlockTokens - 1) / kBlockTokens;  // (of one sequence: the grid's second size)
    const size_t sums_lds = sizeof(float) * (2 * static_cast<size_t>(kBlockTokens) * (padded + 4) +
                                             kBlockTokens * panel_stride(cols16 < kPanelCols ? cols16 : kPanelCols) +
                                             kBlockTokens * kScoreStride + kBlockTokens + 4);
    const size_t reads_lds = sizeof(float) * (static_cast<size_t>(kBlockTokens) * (padded + 4) + kBlockTokens + 4);
    if (sums_lds > 64 * 1024 || most_blocks > 65535 || panels > 65535 || static_cast<long>(sequences) * heads > 0x7fffffffL)
        return CIE_BAD_ARGUMENT;
    if (sequences == 0 || tokens == 0) return CIE_OK;
    BlockArgs a{log_decay, ld_decay, in, ld_in, out, ld_out, heads_per_group, val, ld_val, val_scale, ld_scale, skip,
                state, seq_slot, q_start_loc, y, sums, totals, heads, rows, cols, padded, cols16};
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 block_grid(sequences * heads, most_blocks, panels);
    walk_block_sums_kernel<<<block_grid, 256, sums_lds, s>>>(a);
    if (hipGetLastError() != hipSuccess) return CIE_LAUNCH_FAILED;
    const dim3 scan_grid(sequences * heads, (padded * cols16 + 255) / 256);
    walk_scan_kernel<<<scan_grid, 256, 0, s>>>(a);
    if (hipGetLastError() != hipSuccess) return CIE_LAUNCH_FAILED;
    walk_block_reads_kernel<<<block_grid, 256, reads_lds, s>>>(a);
    return cie_after_launch();
}

CIE_API int cie_space_steps(void* stream, int dtype, const void* raw, long ld, const float* bias, const float* a_log,
                            float* steps, float* decay, float* log_decay, int tokens, int heads) {
    if (tokens < 0 || heads <= 0 || ld < heads || !bias || !a_log || !steps || !decay || !log_decay) return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    const long count = static_cast<long>(tokens) * heads;
    const unsigned blocks = static_cast<unsigned>((count + 255) / 256);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == CIE_F32)
        space_steps_kernel<float><<<blocks, 256, 0, s>>>(static_cast<const float*>(raw), ld, bias, a_log, steps, decay, log_decay, count, heads);
    else if (dtype == CIE_BF16)
        space_steps_kernel<bf16_t><<<blocks, 256, 0, s>>>(static_cast<const bf16_t*>(raw), ld, bias, a_log, steps, decay, log_decay, count, heads);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}

CIE_API int cie_shift_mix(void* stream, int dtype, const void* h, long ldh, const float* before, const float* mu,
                          const int* seq_of_token, const int* seq_slot, const int* q_start_loc, void* mixes, int tokens,
                          int width, int n_mix) {
    if (tokens < 0 || width <= 0 || n_mix <= 0 || ldh < width || !before || !mu) return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int blocks = (width + 255) / 256;
    const dim3 grid(tokens, tokens >= 512 ? 1 : (blocks < 32 ? blocks : 32));
    if (dtype == CIE_F32)
        shift_mix_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(h), ldh, before, mu, seq_of_token, seq_slot,
                                                      q_start_loc, static_cast<float*>(mixes), tokens, width, n_mix);
    else if (dtype == CIE_BF16)
        shift_mix_kernel<bf16_t><<<grid, 256, 0, s>>>(static_cast<const bf16_t*>(h), ldh, before, mu, seq_of_token, seq_slot,
                                                       q_start_loc, static_cast<bf16_t*>(mixes), tokens, width, n_mix);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}

CIE_API int cie_time_decay(void* stream, int dtype, const float* low, const void* w2t, const float* w0, float* decay,
                           int tokens, int channels, int rank, const void* h, long ldh, float* before,
                           const int* seq_of_token, const int* seq_slot, const int* q_start_loc, int width) {
    if (tokens < 0 || channels <= 0 || rank <= 0 || rank > 8192 || width <= 0 || ldh < width || !low || !w2t || !w0 ||
        !decay || !h || !before)
        return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t lds = static_cast<size_t>(rank) * sizeof(float);
    const int most = channels > width ? channels : width;
    const int blocks = (most + 255) / 256;
    const dim3 grid(tokens, tokens >= 512 ? (blocks < 2 ? blocks : 2) : (blocks < 32 ? blocks : 32));
    if (dtype == CIE_F32)
        time_decay_kernel<float><<<grid, 256, lds, s>>>(low, static_cast<const float*>(w2t), w0, decay, channels, rank,
                                                         static_cast<const float*>(h), ldh, before, seq_of_token,
                                                         seq_slot, q_start_loc, width);
    else if (dtype == CIE_BF16)
        time_decay_kernel<bf16_t><<<grid, 256, lds, s>>>(low, static_cast<const bf16_t*>(w2t), w0, decay, channels, rank,
                                                          static_cast<const bf16_t*>(h), ldh, before, seq_of_token,
                                                          seq_slot, q_start_loc, width);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}

CIE_API int cie_gated_group_norm(void* stream, int dtype, const float* y, const void* gate, long ldg,
                                 const float* weight, void* out, int tokens, int width, int groups, float eps,
                                 int gate_first) {
    if (tokens < 0 || width <= 0 || groups <= 0 || width % groups || !(eps > 0.f) || !y || !out ||
        (gate && ldg < width) || (static_cast<size_t>(width) + groups) * sizeof(float) > 64 * 1024)
        return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int threads = width >= 2048 ? 1024 : width >= 1024 ? 512 : 256;
    const size_t lds = (static_cast<size_t>(width) + groups) * sizeof(float);
    if (dtype == CIE_F32)
        gated_group_norm_kernel<float><<<tokens, threads, lds, s>>>(y, static_cast<const float*>(gate), ldg, weight,
                                                                 static_cast<float*>(out), width, groups, eps, gate_first);
    else if (dtype == CIE_BF16)
        gated_group_norm_kernel<bf16_t><<<tokens, threads, lds, s>>>(y, static_cast<const bf16_t*>(gate), ldg, weight,
                                                                  static_cast<bf16_t*>(out), width, groups, eps, gate_first);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}
