// Mixers that carry a state of fixed size from token to token instead of a growing cache.  Every state lives in
// float32 rows of a state tensor, one row per request slot; a step reads the row its earlier steps left, runs its
// tokens in order and writes the row back, so a sequence may be cut into steps anywhere.
//
// 1. retention: a memory S [dim, vdim] per head that fades by a fixed factor per token,
//        S_t = decay * S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,
//    q and k turned by the token's position (the first `rot` dimensions of a head, pair (i, i + rot/2)), k scaled
//    after the turn; o_t divided by its root mean square over the head and multiplied by silu(gate).
// 2. a causal convolution over each channel's own last `taps` inputs, the inputs of the tokens before the step taken
//    from the state.
// 3. a gated linear recurrence per channel,
//        a = exp(c * sigmoid(r)),  S_t = a * S_(t-1) + sqrt(1 - a^2) * sigmoid(i) * u_t,   out_t = S_t * gelu(y_t),
//    with c = -8 softplus(lambda) < 0 made once per model; it also moves the convolution's state on.
//
// Sequence s of the step brings tokens q_start_loc[s] .. q_start_loc[s + 1] - 1 of the flat token axis, the first at
// position seq_start[s]; its state row is seq_slot[s].
#include "common.h"

namespace {

__device__ __forceinline__ float sigmoidf(float x) { return 1.0f / (1.0f + expf(-x)); }

// what stands between a projection and the memory: 0 nothing, 1 silu
__device__ __forceinline__ float activated(float z, int act) { return act == 1 ? z * sigmoidf(z) : z; }

__device__ __forceinline__ float gelu_tanh(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// ---------------------------------------------------------------------------------------------- retention
// Three kernels.  (a) Every token's queries and keys, turned by its position, the keys scaled, as float32 rows padded
// with zeros to `padded` numbers per head: [tokens, heads, 2, padded] (what passes through an activation on its way in
// does so here).  (b) The walk over the tokens, below, token by token for steps of few tokens a sequence, or (b') in
// blocks on the matrix cores for prompts' portions.  (c) The norm over a head's or over several heads' read-outs, the
// norm's weight and the gate, which need all value columns of the heads that share a root mean square.
//
// (b) A column of the memory never meets another column, and o_t is a sum over the memory's rows, so one workgroup
// takes (sequence, head, slice of up to 64 value columns, part of the rows) and the parts' shares of o_t are added
// up by (c): as many parts as give every compute unit a workgroup (a prompt of one sequence with 8 heads of 128 x 256
// would otherwise keep 32 of 256 units busy, each walking its 2,048 tokens at 64 multiply-adds per thread and token).
// Thread (column v, group g) keeps rows r0 + g * DS .. + DS - 1 of column v in registers.  Tokens go in chunks:
// the chunk's queries, keys and values are staged in LDS, every thread walks the chunk's tokens in order (no
// barrier between tokens; a thread reads its DS numbers of a query as 16-byte pieces), and the groups' shares are
// summed into the part's float32 plane [tokens, heads * vdim].  The next chunk's numbers are fetched into
// registers before the walk over the current one starts, so that their way from memory is hidden behind it.
template <typename T>
__global__ void __launch_bounds__(256)
retention_turn_kernel(const T* __restrict__ proj, long ldp, int q_off, int k_off, const float* __restrict__ cos_table,
                      const float* __restrict__ sin_table, int rot, const int* __restrict__ positions,
                      float* __restrict__ turned, int heads, int dim, int padded, float key_scale, int act) {
    const int token = blockIdx.x;
    const int half = rot / 2;
    const T* row = proj + static_cast<size_t>(token) * ldp;
    const size_t at = static_cast<size_t>(positions[token]) * half;
    // (few tokens: the workgroups of a token, blockIdx.y, share its heads' numbers)
    for (int idx = blockIdx.y * blockDim.x + threadIdx.x; idx < heads * padded; idx += blockDim.x * gridDim.y) {
        const int head = idx / padded;
        const int d = idx - head * padded;
        float qv = 0.f, kv = 0.f;
        if (d < dim) {
            const T* qh = row + q_off + head * dim;
            const T* kh = row + k_off + head * dim;
            qv = activated(to_float(qh[d]), act);
            kv = activated(to_float(kh[d]), act);
            if (d < rot) {
                const int i = d < half ? d : d - half;
                const float c = cos_table[at + i], s = sin_table[at + i];
                if (d < half) {
                    qv = qv * c - activated(to_float(qh[d + half]), act) * s;
                    kv = kv * c - activated(to_float(kh[d + half]), act) * s;
                } else {
                    qv = qv * c + activated(to_float(qh[i]), act) * s;
                    kv = kv * c + activated(to_float(kh[i]), act) * s;
                }
            }
        }
        float* dst = turned + ((static_cast<size_t>(token) * heads + head) * 2) * padded + d;
        dst[0] = qv;
        dst[padded] = kv * key_scale;
    }
}

typedef float piece_t __attribute__((ext_vector_type(4)));  // 16 bytes that stay in registers (as a struct of four
                                                            // floats, the pieces fetched ahead went through scratch memory)

constexpr int kFetchPieces = 6;  // 16-byte pieces of a chunk's queries and keys that a thread fetches ahead
constexpr int kFetchValues = 12; // ... and values

// the chunk that starts at token `from`: this thread's pieces into its registers.  Every load stands in straight-line
// code without a condition (a piece or value past the chunk's end reads the chunk's last one again, a column past the
// head's last its last): behind a load under a condition the compiler waits for it before it issues the next, and
// the eighteen loads of a thread became eighteen round trips to memory per chunk.
#define CIE_RETENTION_FETCH(from)                                                                                     \
    {                                                                                                                 \
        const int fetch_n = min(chunk, count - (from));                                                               \
        _Pragma("unroll") for (int i = 0; i < kFetchPieces; ++i) {                                                    \
            const int idx = min(static_cast<int>(threadIdx.x + i * blockDim.x), fetch_n * pieces - 1);                \
            const int t = idx / pieces;                                                                               \
            const int piece = idx - t * pieces;                                                                       \
            const int side = piece / (rows / 4); /* 0: the query, 1: the key */                                       \
            ahead[i] = *reinterpret_cast<const piece_t*>(                                                             \
                turned + ((static_cast<size_t>(first + (from) + t) * heads + head) * 2 + side) * padded + r0 +        \
                (piece - side * (rows / 4)) * 4);                                                                     \
        }                                                                                                             \
        _Pragma("unroll") for (int i = 0; i < kFetchValues; ++i) {                                                    \
            const int idx = min(static_cast<int>(threadIdx.x + i * blockDim.x), fetch_n * slice - 1);                 \
            const int t = idx / slice;                                                                                \
            const int c = min(v0 + idx - t * slice, vdim - 1);                                                        \
            ahead_v[i] = proj[static_cast<size_t>(first + (from) + t) * ldp + v_off + head * vdim + c];               \
        }                                                                                                             \
    }

template <typename T, int DS>
__global__ void __launch_bounds__(512)
retention_kernel(const T* __restrict__ proj, long ldp, int v_off, const float* __restrict__ turned,
                 const float* __restrict__ decay, float* __restrict__ state, const int* __restrict__ seq_slot,
                 const int* __restrict__ q_start_loc, float* __restrict__ raw, long plane,
                 int heads, int dim, int vdim, int slice, int slices, int groups, int padded, int chunk, int act) {
    extern __shared__ float4 lds4[];
    float* lds = reinterpret_cast<float*>(lds4);
    const int rows = groups * DS;              // rows of the memory that this workgroup keeps
    float* qk_s = lds;                         // [chunk][2][rows]: a token's query, then its key
    float* v_s = qk_s + chunk * 2 * rows;      // [chunk][slice]
    float* o_s = v_s + chunk * slice;          // [groups][chunk][slice]
    const int seq = blockIdx.x;
    const int head = blockIdx.y;
    const int part = blockIdx.z / slices;
    const int v0 = (blockIdx.z - part * slices) * slice;
    const int r0 = part * rows;
    const int first = q_start_loc[seq];
    const int count = q_start_loc[seq + 1] - first;
    const int slot = seq_slot[seq];
    const int col = threadIdx.x % slice;
    const int grp = threadIdx.x / slice;
    const bool owner = grp < groups && v0 + col < vdim;
    const int d0 = r0 + grp * DS;
    const float fade = decay[head];
    const int pieces = 2 * rows / 4;           // 16-byte pieces of one token's query and key rows
    float* mem = state + ((static_cast<size_t>(slot) * heads + head) * dim) * vdim + v0 + col;
    float* mine = raw + static_cast<size_t>(part) * plane;
    float S[DS];
#pragma unroll
    for (int r = 0; r < DS; ++r) S[r] = (owner && d0 + r < dim) ? mem[static_cast<size_t>(d0 + r) * vdim] : 0.f;
    piece_t ahead[kFetchPieces];
    T ahead_v[kFetchValues];  // (as stored: a conversion right behind the load would wait for it, and for all loads before it)
    if (count > 0) CIE_RETENTION_FETCH(0)
    for (int c0 = 0; c0 < count; c0 += chunk) {
        const int cn = min(chunk, count - c0);
#pragma unroll
        for (int i = 0; i < kFetchPieces; ++i) {
            const int idx = threadIdx.x + i * blockDim.x;
            if (idx < cn * pieces) reinterpret_cast<piece_t*>(qk_s)[idx] = ahead[i];
        }
#pragma unroll
        for (int i = 0; i < kFetchValues; ++i) {
            const int idx = threadIdx.x + i * blockDim.x;
            if (idx < cn * slice) v_s[idx] = activated(to_float(ahead_v[i]), act);
        }
        __syncthreads();
        if (c0 + chunk < count) CIE_RETENTION_FETCH(c0 + chunk)
        if (owner) {
            // (a token's numbers are read from LDS while the token before it is worked on: with one wave per SIMD
            // nothing else would hide the way from LDS, and it is as long as the arithmetic of a token)
            const float* q_base = qk_s + grp * DS;
            float4 q_next[DS / 4], k_next[DS / 4];
            float v_next = v_s[col];
#pragma unroll
            for (int r = 0; r < DS / 4; ++r) {
                q_next[r] = reinterpret_cast<const float4*>(q_base)[r];
                k_next[r] = reinterpret_cast<const float4*>(q_base + rows)[r];
            }
            for (int t = 0; t < cn; ++t) {
                float4 q_now[DS / 4], k_now[DS / 4];
                const float vt = v_next;
#pragma unroll
                for (int r = 0; r < DS / 4; ++r) {
                    q_now[r] = q_next[r];
                    k_now[r] = k_next[r];
                }
                const int ahead_t = min(t + 1, cn - 1);  // (the last token is read twice: no condition around the reads)
                v_next = v_s[ahead_t * slice + col];
#pragma unroll
                for (int r = 0; r < DS / 4; ++r) {
                    q_next[r] = reinterpret_cast<const float4*>(q_base + ahead_t * 2 * rows)[r];
                    k_next[r] = reinterpret_cast<const float4*>(q_base + ahead_t * 2 * rows + rows)[r];
                }
                float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
                for (int r = 0; r < DS / 4; ++r) {
                    const float4 k4 = k_now[r], q4 = q_now[r];
                    S[4 * r + 0] = fmaf(fade, S[4 * r + 0], k4.x * vt);
                    S[4 * r + 1] = fmaf(fade, S[4 * r + 1], k4.y * vt);
                    S[4 * r + 2] = fmaf(fade, S[4 * r + 2], k4.z * vt);
                    S[4 * r + 3] = fmaf(fade, S[4 * r + 3], k4.w * vt);
                    a0 = fmaf(S[4 * r + 0], q4.x, a0);
                    a1 = fmaf(S[4 * r + 1], q4.y, a1);
                    a2 = fmaf(S[4 * r + 2], q4.z, a2);
                    a3 = fmaf(S[4 * r + 3], q4.w, a3);
                }
                o_s[(grp * chunk + t) * slice + col] = (a0 + a1) + (a2 + a3);
            }
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < cn * slice; idx += blockDim.x) {
            const int t = idx / slice;
            const int c = idx - t * slice;
            if (v0 + c >= vdim) continue;
            float o = 0.f;
            for (int g = 0; g < groups; ++g) o += o_s[(g * chunk + t) * slice + c];
            mine[static_cast<size_t>(first + c0 + t) * heads * vdim + head * vdim + v0 + c] = o;
        }
        __syncthreads();
    }
    if (owner)
#pragma unroll
        for (int r = 0; r < DS; ++r)
            if (d0 + r < dim) mem[static_cast<size_t>(d0 + r) * vdim] = S[r];
}
#undef CIE_RETENTION_FETCH

// (b') The same walk for sequences that bring many tokens (a prompt's portion): blocks of 32 tokens on the matrix
// cores, float32 throughout (`v_mfma_f32_16x16x4_f32`: operands and sums are plain float32), and only what has to
// wait for the block before it waits.  With S the memory in front of a block of n tokens, i and j tokens of the
// block and f the head's decay:
//     o_i   = f^(i+1) * (S^T q_i)  +  sum_{j <= i} f^(i-j) (q_i . k_j) v_j
//     S_new = f^n * S  +  sum_j f^(n-1-j) k_j v_j^T
// Three kernels.  `retention_block_sums_kernel`, every block at once: the second term of o (into the first plane of
// `raw`) and the second term of S_new (into the block's place of `sums`).  `retention_scan_kernel`, one thread per
// number of the memory, over a sequence's blocks in order: the block's place gets the S in front of it, and S moves on.
// `retention_block_reads_kernel`, every block at once: the first term of o (into the second plane).  The norm kernel
// adds the planes.  Block b of sequence s has place first_token(s) / 32 + s + b: no two blocks share one, and there
// are at most tokens / 32 + sequences + 1 places.  Queries and keys are the turn kernel's float32 rows, padded to whole
// tiles of 16; a workgroup takes up to 128 value columns (a panel), rounded up to tiles of 16 (`vdim16` columns a row
// of `sums`).  Operand layouts of the 16 x 16 x 4 product: lane (l16 = lane % 16, g = lane / 16) gives A[l16][g] and
// B[g][l16] and gets rows 4 g .. 4 g + 3 of column l16; which four numbers of a sum a product takes does not matter
// as long as both operands agree, so a lane reads four neighbouring numbers at once and spends them on four products.
typedef float acc4_t __attribute__((ext_vector_type(4)));
constexpr int kBlockTokens = 32;
constexpr int kPanelCols = 128;
constexpr int kScoreStride = kBlockTokens + 4;

// rows of a panel of values in LDS start 16 banks apart: the four tokens that a product reads then touch every bank
__host__ __device__ inline int panel_stride(int cols) { return cols % 32 == 0 ? cols + 16 : cols; }

// powers of the decay by repeated multiplication, as the walk token by token makes them
__device__ __forceinline__ void decay_table(float* pw, float fade) {
    if (threadIdx.x == 0) {
        float f = 1.0f;
        for (int n = 0; n <= kBlockTokens; ++n) {
            pw[n] = f;
            f *= fade;
        }
    }
}

// a block's queries (side 0) or keys (side 1) into LDS rows of `stride` floats; rows past the block's last token are zero
__device__ __forceinline__ void stage_rows(float* dst, int stride, const float* __restrict__ turned, int first_token,
                                           int cn, int heads, int head, int padded, int side) {
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    for (int t = wave; t < kBlockTokens; t += 4) {
        const float* src = turned + ((static_cast<size_t>(first_token + min(t, cn - 1)) * heads + head) * 2 + side) * padded;
        for (int piece = lane; piece < padded / 4; piece += kWave) {
            const piece_t value = *reinterpret_cast<const piece_t*>(src + 4 * piece);
            *reinterpret_cast<piece_t*>(dst + t * stride + 4 * piece) = t < cn ? value : piece_t{0.f, 0.f, 0.f, 0.f};
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(256)
retention_block_sums_kernel(const T* __restrict__ proj, long ldp, int v_off, const float* __restrict__ turned,
                            const float* __restrict__ decay, const int* __restrict__ q_start_loc,
                            float* __restrict__ raw, float* __restrict__ sums, int heads, int vdim, int padded,
                            int vdim16, int act) {
    const int seq = blockIdx.x / heads;
    const int head = blockIdx.x - seq * heads;
    const int first = q_start_loc[seq];
    const int count = q_start_loc[seq + 1] - first;
    const int c0 = blockIdx.y * kBlockTokens;
    if (c0 >= count) return;                             // (the whole workgroup: the grid is sized for the longest sequence)
    const int cn = min(kBlockTokens, count - c0);
    const int panel0 = blockIdx.z * kPanelCols;
    const int cols = min(kPanelCols, vdim16 - panel0);
    const int col_tiles = cols / 16;
    const int stride = padded + 4;
    const int vstride = panel_stride(cols);
    extern __shared__ float4 lds4[];
    float* q_s = reinterpret_cast<float*>(lds4);          // [32][stride]
    float* k_s = q_s + kBlockTokens * stride;            // [32][stride]
    float* v_s = k_s + kBlockTokens * stride;            // [32][vstride]
    float* p_s = v_s + kBlockTokens * vstride;           // [32][36]: f^(i-j) (q_i . k_j), zero above the diagonal
    float* pw = p_s + kBlockTokens * kScoreStride;       // [33]
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int l16 = lane % 16;
    const int g = lane / 16;
    const int tiles = padded / 16;
    decay_table(pw, decay[head]);
    stage_rows(q_s, stride, turned, first + c0, cn, heads, head, padded, 0);
    stage_rows(k_s, stride, turned, first + c0, cn, heads, head, padded, 1);
    for (int t = wave; t < kBlockTokens; t += 4) {
        const T* src = proj + static_cast<size_t>(first + c0 + min(t, cn - 1)) * ldp + v_off + head * vdim;
        for (int c = lane; c < cols; c += kWave) {
            const float value = activated(to_float(src[min(panel0 + c, vdim - 1)]), act);
            v_s[t * vstride + c] = (t < cn && panel0 + c < vdim) ? value : 0.f;
        }
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
                const float4 a = *reinterpret_cast<const float4*>(qa + 16 * m);
                const float4 b = *reinterpret_cast<const float4*>(kb + 16 * m);
                p = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b.x, p, 0, 0, 0);
                p1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b.y, p1, 0, 0, 0);
                p = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b.z, p, 0, 0, 0);
                p1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b.w, p1, 0, 0, 0);
            }
            p += p1;
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int apart = 16 * (ti - tj) + 4 * g + r - l16;  // i - j
            p_s[(16 * ti + 4 * g + r) * kScoreStride + 16 * tj + l16] = apart >= 0 ? p[r] * pw[min(apart, kBlockTokens)] : 0.f;
        }
    }
    __syncthreads();
    float k_fade[kBlockTokens / 4];
#pragma unroll
    for (int kk = 0; kk < kBlockTokens / 4; ++kk) k_fade[kk] = pw[max(cn - 1 - (4 * kk + g), 0)];
    const int place = first / kBlockTokens + seq + blockIdx.y;
    float* sum_rows = sums + (static_cast<size_t>(place) * heads + head) * padded * vdim16 + panel0;
    for (int ct = wave; ct < col_tiles; ct += 4) {       // this wave's tiles of value columns
        float vb[kBlockTokens / 4];
#pragma unroll
        for (int kk = 0; kk < kBlockTokens / 4; ++kk) vb[kk] = v_s[(4 * kk + g) * vstride + 16 * ct + l16];
        // the block's own sum
        acc4_t o0 = {0.f, 0.f, 0.f, 0.f}, o1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < kBlockTokens / 4; ++kk) {
            o0 = __builtin_amdgcn_mfma_f32_16x16x4f32(p_s[l16 * kScoreStride + 4 * kk + g], vb[kk], o0, 0, 0, 0);
            o1 = __builtin_amdgcn_mfma_f32_16x16x4f32(p_s[(16 + l16) * kScoreStride + 4 * kk + g], vb[kk], o1, 0, 0, 0);
        }
        const int col = panel0 + 16 * ct + l16;
        if (col < vdim) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = 4 * g + r;
                float* dst = raw + static_cast<size_t>(first + c0) * heads * vdim + head * vdim + col;
                if (i < cn) dst[static_cast<size_t>(i) * heads * vdim] = o0[r];
                if (16 + i < cn) dst[static_cast<size_t>(16 + i) * heads * vdim] = o1[r];
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
            for (int r = 0; r < 4; ++r) sum_rows[static_cast<size_t>(16 * rt + 4 * g + r) * vdim16 + 16 * ct + l16] = acc[r];
        }
    }
}

// One thread per number of a head's memory (rows and columns padded as `sums` has them): over the sequence's blocks in
// order, the block's place gets the memory in front of the block, and the memory moves on by the block's sum.
__global__ void __launch_bounds__(256)
retention_scan_kernel(const float* __restrict__ decay, float* __restrict__ state, const int* __restrict__ seq_slot,
                      const int* __restrict__ q_start_loc, float* __restrict__ sums, int heads, int dim, int vdim,
                      int padded, int vdim16) {
    const int seq = blockIdx.x / heads;
    const int head = blockIdx.x - seq * heads;
    const int e = blockIdx.y * blockDim.x + threadIdx.x;
    if (e >= padded * vdim16) return;
    const int first = q_start_loc[seq];
    const int count = q_start_loc[seq + 1] - first;
    if (count <= 0) return;
    const int row = e / vdim16;
    const int col = e - row * vdim16;
    const bool real = row < dim && col < vdim;
    float* mem = state + ((static_cast<size_t>(seq_slot[seq]) * heads + head) * dim + row) * vdim + col;
    float S = real ? *mem : 0.f;
    const int blocks = (count + kBlockTokens - 1) / kBlockTokens;
    const float fade = decay[head];
    float whole = 1.0f, rest = 1.0f;
    for (int n = 0; n < kBlockTokens; ++n) whole *= fade;
    for (int n = 0; n < count - (blocks - 1) * kBlockTokens; ++n) rest *= fade;
    const size_t step = static_cast<size_t>(heads) * padded * vdim16;
    float* at = sums + (static_cast<size_t>(first / kBlockTokens + seq) * heads + head) * padded * vdim16 + e;
    float add = at[0];
    for (int b = 0; b < blocks; ++b) {
        const float next = at[static_cast<size_t>(min(b + 1, blocks - 1)) * step];  // (asked for before this block's place is written)
        at[static_cast<size_t>(b) * step] = S;
        S = (b == blocks - 1 ? rest : whole) * S + add;
        add = next;
    }
    if (real) *mem = S;
}

__global__ void __launch_bounds__(256)
retention_block_reads_kernel(const float* __restrict__ turned, const float* __restrict__ decay,
                             const int* __restrict__ q_start_loc, const float* __restrict__ sums, float* __restrict__ raw,
                             int heads, int vdim, int padded, int vdim16) {
    const int seq = blockIdx.x / heads;
    const int head = blockIdx.x - seq * heads;
    const int first = q_start_loc[seq];
    const int count = q_start_loc[seq + 1] - first;
    const int c0 = blockIdx.y * kBlockTokens;
    if (c0 >= count) return;
    const int cn = min(kBlockTokens, count - c0);
    const int panel0 = blockIdx.z * kPanelCols;
    const int col_tiles = min(kPanelCols, vdim16 - panel0) / 16;
    const int stride = padded + 4;
    extern __shared__ float4 lds4[];
    float* q_s = reinterpret_cast<float*>(lds4);          // [32][stride]
    float* pw = q_s + kBlockTokens * stride;             // [33]
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int l16 = lane % 16;
    const int g = lane / 16;
    const int tiles = padded / 16;
    decay_table(pw, decay[head]);
    stage_rows(q_s, stride, turned, first + c0, cn, heads, head, padded, 0);
    __syncthreads();
    const int place = first / kBlockTokens + seq + blockIdx.y;
    const float* before = sums + (static_cast<size_t>(place) * heads + head) * padded * vdim16 + panel0;
    for (int ct = wave; ct < col_tiles; ct += 4) {
        acc4_t o0 = {0.f, 0.f, 0.f, 0.f}, o1 = {0.f, 0.f, 0.f, 0.f};
        const float* rows = before + static_cast<size_t>(4 * g) * vdim16 + 16 * ct + l16;
#pragma unroll 2
        for (int m = 0; m < tiles; ++m) {
            const float4 a0 = *reinterpret_cast<const float4*>(q_s + l16 * stride + 16 * m + 4 * g);
            const float4 a1 = *reinterpret_cast<const float4*>(q_s + (16 + l16) * stride + 16 * m + 4 * g);
            const float* s = rows + static_cast<size_t>(16 * m) * vdim16;
            const float b0 = s[0], b1 = s[vdim16], b2 = s[2 * vdim16], b3 = s[3 * vdim16];
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
        if (col < vdim) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = 4 * g + r;
                float* dst = raw + static_cast<size_t>(first + c0) * heads * vdim + head * vdim + col;
                if (i < cn) dst[static_cast<size_t>(i) * heads * vdim] = o0[r] * pw[i + 1];
                if (16 + i < cn) dst[static_cast<size_t>(16 + i) * heads * vdim] = o1[r] * pw[16 + i + 1];
            }
        }
    }
}

// o / sqrt(mean(o^2) + eps) [* weight] * gate: one wave per (token, run of `span` heads).  The mean runs over the
// `span` heads of a run together (1: every head by itself; `heads`: all of a token's heads as one vector); `weight`
// [heads * vdim] float32 or null; the gate is silu(g) (gate_act 0) or sigmoid(g) (1) of the projection's gate columns.
template <typename T>
__global__ void __launch_bounds__(256)
retention_norm_kernel(float* __restrict__ raw, long plane, int parts, const T* __restrict__ proj, long ldp, int g_off,
                      T* __restrict__ out, int tokens, int heads, int vdim, float eps, int span,
                      const float* __restrict__ weight, int gate_act) {
    const int runs = heads / span;
    const int item = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
    if (item >= tokens * runs) return;  // (whole waves leave together)
    const int lane = threadIdx.x % kWave;
    const int token = item / runs;
    const int first = (item - token * runs) * span * vdim;  // the run's first column
    const int width = span * vdim;
    float* o = raw + static_cast<size_t>(token) * heads * vdim + first;
    float sum_sq = 0.f;
    for (int c = lane; c < width; c += kWave) {
        float v = o[c];
        for (int p = 1; p < parts; ++p) v += o[static_cast<size_t>(p) * plane + c];  // (the parts in their order)
        o[c] = v;  // (this lane's own column: it reads it again below)
        sum_sq += v * v;
    }
    const float inv = 1.0f / sqrtf(wave_sum(sum_sq) / static_cast<float>(width) + eps);
    const T* gate = proj + static_cast<size_t>(token) * ldp + g_off + first;
    T* dst = out + static_cast<size_t>(token) * heads * vdim + first;
    for (int c = lane; c < width; c += kWave) {
        const float g = to_float(gate[c]);
        const float open = gate_act == 1 ? sigmoidf(g) : g * sigmoidf(g);
        float y = o[c] * inv;
        if (weight) y *= weight[first + c];
        dst[c] = from_float<T>(y * open);
    }
}

// The same for runs wider than a wave takes well (a norm over all heads of a token): one workgroup per (token, run),
// the summed columns wait in LDS, the waves' sums of squares meet there in the waves' order.
template <typename T>
__global__ void __launch_bounds__(1024)
retention_norm_wide_kernel(const float* __restrict__ raw, long plane, int parts, const T* __restrict__ proj, long ldp,
                           int g_off, T* __restrict__ out, int heads, int vdim, float eps, int span,
                           const float* __restrict__ weight, int gate_act) {
    extern __shared__ float wide[];  // [span * vdim] the run's columns, then one sum of squares per wave
    const int runs = heads / span;
    const int token = blockIdx.x / runs;
    const int first = (blockIdx.x - token * runs) * span * vdim;
    const int width = span * vdim;
    float* partial = wide + width;
    const float* o = raw + static_cast<size_t>(token) * heads * vdim + first;
    float sum_sq = 0.f;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        float v = o[c];
        for (int p = 1; p < parts; ++p) v += o[static_cast<size_t>(p) * plane + c];  // (the parts in their order)
        wide[c] = v;  // (this thread's own column: it reads it again below)
        sum_sq += v * v;
    }
    sum_sq = wave_sum(sum_sq);
    if (threadIdx.x % kWave == 0) partial[threadIdx.x / kWave] = sum_sq;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < static_cast<int>(blockDim.x) / kWave; ++w) total += partial[w];
    const float inv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
    const T* gate = proj + static_cast<size_t>(token) * ldp + g_off + first;
    T* dst = out + static_cast<size_t>(token) * heads * vdim + first;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        const float g = to_float(gate[c]);
        const float open = gate_act == 1 ? sigmoidf(g) : g * sigmoidf(g);
        float y = wide[c] * inv;
        if (weight) y *= weight[first + c];
        dst[c] = from_float<T>(y * open);
    }
}

template <typename T, int DS>
int launch_retention(hipStream_t s, dim3 grid, int threads, size_t lds, const void* proj, long ldp, int v_off,
                     const float* turned, const float* decay, float* state, const int* seq_slot, const int* q_start_loc,
                     float* raw, long plane, int heads, int dim, int vdim, int slice, int slices, int groups, int padded,
                     int chunk, int act) {
    retention_kernel<T, DS><<<grid, threads, lds, s>>>(static_cast<const T*>(proj), ldp, v_off, turned, decay, state,
                                                      seq_slot, q_start_loc, raw, plane, heads, dim, vdim, slice, slices,
                                                      groups, padded, chunk, act);
    return cie_after_launch();
}

// ---------------------------------------------------------------------------------------------- convolution
// (`act`: what the sum passes through, 0 nothing, 1 silu; O: the type it is stored in)
template <typename T, typename O>
__global__ void __launch_bounds__(256)
causal_conv_kernel(const T* __restrict__ x, long ldx, const T* __restrict__ taps_w, const T* __restrict__ bias,
                   const float* __restrict__ past, const int* __restrict__ seq_of_token, const int* __restrict__ seq_slot,
                   const int* __restrict__ q_start_loc, O* __restrict__ out, int channels, int taps, int act) {
    const int token = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int seq = seq_of_token[token];
    const int first = q_start_loc[seq];
    const int t = token - first;
    const float* before = past + static_cast<size_t>(seq_slot[seq]) * max(taps - 1, 1) * channels;
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
        const int src = t - (taps - 1) + j;  // the last tap is this token's input
        const float in = src >= 0 ? to_float(x[static_cast<size_t>(first + src) * ldx + c])
                                  : before[static_cast<size_t>(taps - 1 + src) * channels + c];
        acc = fmaf(to_float(taps_w[static_cast<size_t>(c) * taps + j]), in, acc);
    }
    if (bias) acc += to_float(bias[c]);
    out[static_cast<size_t>(token) * channels + c] = from_float<O>(activated(acc, act));
}

// The convolution's state moved on by a step's inputs: of [what the state held, the step's inputs] the last
// taps - 1 rows.  One thread per (sequence, channel); runs behind the convolution that still read the old rows.
template <typename T>
__global__ void __launch_bounds__(256)
conv_keep_kernel(const T* __restrict__ x, long ldx, float* __restrict__ past, const int* __restrict__ seq_slot,
                 const int* __restrict__ q_start_loc, int channels, int taps) {
    const int seq = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const int keep_n = taps - 1;
    if (c >= channels || keep_n <= 0) return;
    const int first = q_start_loc[seq];
    const int count = q_start_loc[seq + 1] - first;
    float* before = past + static_cast<size_t>(seq_slot[seq]) * keep_n * channels;
    float old[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) old[j] = j < keep_n ? before[static_cast<size_t>(j) * channels + c] : 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        if (j >= keep_n) break;
        const int src = count + j;  // index into [old (keep_n), new (count)]
        before[static_cast<size_t>(j) * channels + c] =
            src < keep_n ? old[src < 16 ? src : 0] : to_float(x[static_cast<size_t>(first + src - keep_n) * ldx + c]);
    }
}

// ---------------------------------------------------------------------------------------------- gated recurrence
// S_t = a_t S_(t-1) + x_t is linear in S, so a sequence's tokens are cut into `segments` stretches that run side by
// side: thread (channel, stretch) first folds its stretch into (A, B) with S_out = A S_in + B, the stretches before
// it give its S_in (a chain of at most `segments` multiply-adds), and a second walk over the stretch makes the
// outputs.  With one stretch this is the plain walk in order.  16 channels per workgroup when cut into stretches.
constexpr int kMaxTaps = 16;
constexpr int kMaxSegments = 16;

// (kScanChannels channels a workgroup: 64 for the walk in order; 16 when cut into stretches, where the arithmetic per
// token bounds the kernel and more workgroups mean more compute units at work)
template <typename T, int kScanChannels>
__global__ void __launch_bounds__(kScanChannels == 64 ? 64 : kScanChannels * kMaxSegments)
gated_recurrence_kernel(const T* __restrict__ y_pre, long ldy, const T* __restrict__ x_in, long ldx,
                        const T* __restrict__ u, const float* __restrict__ gates, int block_width,
                        const float* __restrict__ rate, float* __restrict__ state, float* __restrict__ past,
                        const int* __restrict__ seq_slot, const int* __restrict__ q_start_loc, T* __restrict__ out,
                        int channels, int taps, int segments) {
    __shared__ float a_s[kMaxSegments][kScanChannels];
    __shared__ float b_s[kMaxSegments][kScanChannels];
    const int seq = blockIdx.y;
    const int lane = threadIdx.x % kScanChannels;
    const int seg = threadIdx.x / kScanChannels;
    const int c = blockIdx.x * kScanChannels + lane;
    const bool live = c < channels;
    const int first = q_start_loc[seq];
    const int count = q_start_loc[seq + 1] - first;
    const int slot = seq_slot[seq];
    const int per = (count + segments - 1) / segments;
    const int t0 = min(seg * per, count), t1 = min(t0 + per, count);
    const int block = live ? c / block_width : 0;
    const size_t r_at = static_cast<size_t>(block) * 2 * block_width + (c - block * block_width);
    const size_t i_at = r_at + block_width;
    const float coef = live ? rate[c] : 0.f;
    // a_t and x_t of one token
    auto step = [&](int t, float& a, float& x) {
        const size_t token = static_cast<size_t>(first + t);
        const float r = sigmoidf(gates[token * 2 * channels + r_at]);
        const float i = sigmoidf(gates[token * 2 * channels + i_at]);
        const float log_a = coef * r;
        a = expf(log_a);
        x = sqrtf(-expm1f(2.0f * log_a)) * (i * to_float(u[token * channels + c]));  // sqrt(1 - a^2), no cancellation
    };
    float S = live ? state[static_cast<size_t>(slot) * channels + c] : 0.f;
    if (segments > 1) {
        float A = 1.f, B = 0.f;
        if (live)
#pragma unroll 4
            for (int t = t0; t < t1; ++t) {  // (four tokens per turn: their loads travel together)
                float a, x;
                step(t, a, x);
                B = fmaf(a, B, x);
                A *= a;
            }
        a_s[seg][lane] = A;
        b_s[seg][lane] = B;
        __syncthreads();
        for (int before = 0; before < seg; ++before) S = fmaf(a_s[before][lane], S, b_s[before][lane]);
    }
    if (!live) return;
#pragma unroll 4
    for (int t = t0; t < t1; ++t) {
        float a, x;
        step(t, a, x);
        S = fmaf(a, S, x);
        const size_t token = static_cast<size_t>(first + t);
        out[token * channels + c] = from_float<T>(S * gelu_tanh(to_float(y_pre[token * ldy + c])));
    }
    if (seg != segments - 1) return;
    state[static_cast<size_t>(slot) * channels + c] = S;  // (the last stretch ends where the sequence ends)
    // the convolution's last taps - 1 inputs: those of this step, and behind them what the state held
    const int keep_n = taps - 1;
    if (keep_n <= 0) return;
    float* before = past + static_cast<size_t>(slot) * keep_n * channels;
    float old[kMaxTaps];
#pragma unroll
    for (int j = 0; j < kMaxTaps; ++j) old[j] = j < keep_n ? before[static_cast<size_t>(j) * channels + c] : 0.f;
#pragma unroll
    for (int j = 0; j < kMaxTaps; ++j) {
        if (j >= keep_n) break;
        const int src = count + j;  // index into [old (keep_n), new (count)]
        before[static_cast<size_t>(j) * channels + c] =
            src < keep_n ? old[src < kMaxTaps ? src : 0] : to_float(x_in[static_cast<size_t>(first + src - keep_n) * ldx + c]);
    }
}

}  // namespace

CIE_API int cie_retention(void* stream, int dtype, const void* proj, long ldp, int q_off, int k_off, int v_off, int g_off,
                          const float* cos_table, const float* sin_table, int rot, const float* decay, float* state,
                          const int* seq_slot, const int* positions, const int* q_start_loc, float* turned, float* raw,
                          void* out, int tokens, int sequences, int heads, int dim, int vdim, int rows_per_thread,
                          int groups, int parts, int slice, int chunk, float eps, float key_scale, int act,
                          int norm_span, const float* norm_weight, int gate_act, int blocks, float* sums) {
    if (act < 0 || act > 1 || norm_span < 1 || heads % norm_span || gate_act < 0 || gate_act > 1) return CIE_BAD_ARGUMENT;
    if (blocks) {
        // the walk in blocks on the matrix cores: two planes of o, queries and keys padded to whole tiles of 16
        if (!sums) return CIE_BAD_ARGUMENT;
        groups = 1;
        rows_per_thread = 16;
        parts = (dim + 15) / 16;
        slice = vdim < 16 ? vdim : 16;
        chunk = 1;
    }
    if (sequences < 0 || tokens < 0 || heads <= 0 || heads > 65535 || dim <= 0 || vdim <= 0 || groups <= 0 || chunk <= 0 ||
        parts <= 0 || slice <= 0 || slice > vdim || rot < 0 || rot % 2 || rot > dim ||
        (rot > 0 && (!cos_table || !sin_table)) || !(eps > 0.f) ||
        static_cast<long>(rows_per_thread) * groups * parts < dim || !raw || !turned)
        return CIE_BAD_ARGUMENT;
    const int slices = (vdim + slice - 1) / slice;
    const int threads = ((slice * groups + kWave - 1) / kWave) * kWave;
    const int rows = groups * rows_per_thread;
    const int padded = rows * parts;
    const size_t lds = sizeof(float) * static_cast<size_t>(chunk) *
                       (2 * static_cast<size_t>(rows) + slice + static_cast<size_t>(groups) * slice);
    if (!blocks && (threads > 512 || lds > 64 * 1024 || static_cast<long>(slices) * parts > 65535 ||
                    static_cast<long>(chunk) * 2 * rows / 4 > static_cast<long>(kFetchPieces) * threads ||
                    static_cast<long>(chunk) * slice > static_cast<long>(kFetchValues) * threads))
        return CIE_BAD_ARGUMENT;
    const int vdim16 = (vdim + 15) / 16 * 16;
    const int panels = (vdim16 + kPanelCols - 1) / kPanelCols;
    const int most_blocks = (tokens + kBlockTokens - 1) / kBlockTokens;  // (of one sequence: the grid's second size)
    const size_t sums_lds = sizeof(float) * (2 * static_cast<size_t>(kBlockTokens) * (padded + 4) +
                                             kBlockTokens * panel_stride(vdim16 < kPanelCols ? vdim16 : kPanelCols) +
                                             kBlockTokens * kScoreStride + 36);
    const size_t reads_lds = sizeof(float) * (static_cast<size_t>(kBlockTokens) * (padded + 4) + 36);
    if (blocks && (sums_lds > 64 * 1024 || most_blocks > 65535 || panels > 65535 ||
                   static_cast<long>(sequences) * heads > 0x7fffffffL))
        return CIE_BAD_ARGUMENT;
    if (sequences == 0 || tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // a step of few tokens: up to sixteen workgroups a token, so that a single token's heads do not wait for one
    const int turn_blocks = (heads * padded + 255) / 256;
    const int per_token = tokens >= 256 ? 1 : (turn_blocks < 16 ? turn_blocks : 16);
    const dim3 turn_grid(tokens, per_token);
    if (dtype == CIE_F32)
        retention_turn_kernel<float><<<turn_grid, 256, 0, s>>>(static_cast<const float*>(proj), ldp, q_off, k_off, cos_table,
                                                           sin_table, rot, positions, turned, heads, dim, padded, key_scale, act);
    else if (dtype == CIE_BF16)
        retention_turn_kernel<bf16_t><<<turn_grid, 256, 0, s>>>(static_cast<const bf16_t*>(proj), ldp, q_off, k_off, cos_table,
                                                            sin_table, rot, positions, turned, heads, dim, padded, key_scale, act);
    else
        return CIE_BAD_ARGUMENT;
    const long plane = static_cast<long>(tokens) * heads * vdim;
    int code = CIE_BAD_ARGUMENT;
    if (blocks) {
        const dim3 block_grid(sequences * heads, most_blocks, panels);
        if (dtype == CIE_F32)
            retention_block_sums_kernel<float><<<block_grid, 256, sums_lds, s>>>(
                static_cast<const float*>(proj), ldp, v_off, turned, decay, q_start_loc, raw, sums, heads, vdim, padded,
                vdim16, act);
        else
            retention_block_sums_kernel<bf16_t><<<block_grid, 256, sums_lds, s>>>(
                static_cast<const bf16_t*>(proj), ldp, v_off, turned, decay, q_start_loc, raw, sums, heads, vdim, padded,
                vdim16, act);
        code = cie_after_launch();
        if (code != CIE_OK) return code;
        const dim3 scan_grid(sequences * heads, (padded * vdim16 + 255) / 256);
        retention_scan_kernel<<<scan_grid, 256, 0, s>>>(decay, state, seq_slot, q_start_loc, sums, heads, dim, vdim, padded,
                                                       vdim16);
        code = cie_after_launch();
        if (code != CIE_OK) return code;
        retention_block_reads_kernel<<<block_grid, 256, reads_lds, s>>>(turned, decay, q_start_loc, sums, raw + plane, heads,
                                                                         vdim, padded, vdim16);
        code = cie_after_launch();
        parts = 2;
    } else {
        dim3 grid(sequences, heads, slices * parts);
#define CIE_RETENTION(T, DS)                                                                                         \
        code = launch_retention<T, DS>(s, grid, threads, lds, proj, ldp, v_off, turned, decay, state, seq_slot,          \
                                       q_start_loc, raw, plane, heads, dim, vdim, slice, slices, groups, padded, chunk, act)
        if (dtype == CIE_F32) {
            if (rows_per_thread == 4) CIE_RETENTION(float, 4);
            else if (rows_per_thread == 8) CIE_RETENTION(float, 8);
            else if (rows_per_thread == 16) CIE_RETENTION(float, 16);
            else if (rows_per_thread == 32) CIE_RETENTION(float, 32);
        } else {
            if (rows_per_thread == 4) CIE_RETENTION(bf16_t, 4);
            else if (rows_per_thread == 8) CIE_RETENTION(bf16_t, 8);
            else if (rows_per_thread == 16) CIE_RETENTION(bf16_t, 16);
            else if (rows_per_thread == 32) CIE_RETENTION(bf16_t, 32);
        }
#undef CIE_RETENTION
    }
    if (code != CIE_OK) return code;
    const int items = tokens * (heads / norm_span);
    const int width = norm_span * vdim;
    if (width > 256 && (static_cast<size_t>(width) + 16) * sizeof(float) <= 60 * 1024) {
        // (which kernel norms depends on the run's width alone, never on what else the step holds)
        const int threads = width >= 2048 ? 1024 : width >= 1024 ? 512 : 256;
        const size_t norm_lds = (static_cast<size_t>(width) + 16) * sizeof(float);
        if (dtype == CIE_F32)
            retention_norm_wide_kernel<float><<<items, threads, norm_lds, s>>>(
                raw, plane, parts, static_cast<const float*>(proj), ldp, g_off, static_cast<float*>(out), heads, vdim, eps,
                norm_span, norm_weight, gate_act);
        else
            retention_norm_wide_kernel<bf16_t><<<items, threads, norm_lds, s>>>(
                raw, plane, parts, static_cast<const bf16_t*>(proj), ldp, g_off, static_cast<bf16_t*>(out), heads, vdim,
                eps, norm_span, norm_weight, gate_act);
        return cie_after_launch();
    }
    const int norm_blocks = (items + 3) / 4;
    if (dtype == CIE_F32)
        retention_norm_kernel<float><<<norm_blocks, 256, 0, s>>>(raw, plane, parts, static_cast<const float*>(proj), ldp, g_off,
                                                           static_cast<float*>(out), tokens, heads, vdim, eps, norm_span,
                                                           norm_weight, gate_act);
    else
        retention_norm_kernel<bf16_t><<<norm_blocks, 256, 0, s>>>(raw, plane, parts, static_cast<const bf16_t*>(proj), ldp, g_off,
                                                            static_cast<bf16_t*>(out), tokens, heads, vdim, eps, norm_span,
                                                            norm_weight, gate_act);
    return cie_after_launch();
}

CIE_API int cie_causal_conv(void* stream, int dtype, const void* x, long ldx, const void* taps_w, const void* bias,
                            const float* past, const int* seq_of_token, const int* seq_slot, const int* q_start_loc,
                            void* out, int tokens, int channels, int taps, int act, int out_f32) {
    if (tokens < 0 || tokens > 65535 * 1 || channels <= 0 || taps < 1 || taps > kMaxTaps || ldx < channels || act < 0 ||
        act > 1)
        return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid((channels + 255) / 256, tokens);
#define CIE_CONV(T, O)                                                                                              \
    causal_conv_kernel<T, O><<<grid, 256, 0, s>>>(static_cast<const T*>(x), ldx, static_cast<const T*>(taps_w),          \
                                                  static_cast<const T*>(bias), past, seq_of_token, seq_slot,            \
                                                  q_start_loc, static_cast<O*>(out), channels, taps, act)
    if (dtype == CIE_F32) CIE_CONV(float, float);
    else if (dtype == CIE_BF16 && out_f32) CIE_CONV(bf16_t, float);
    else if (dtype == CIE_BF16) CIE_CONV(bf16_t, bf16_t);
#undef CIE_CONV
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}

// Moves the convolution's state on by the step's inputs (see conv_keep_kernel); call it behind cie_causal_conv.
CIE_API int cie_conv_keep(void* stream, int dtype, const void* x, long ldx, float* past, const int* seq_slot,
                          const int* q_start_loc, int sequences, int channels, int taps) {
    if (sequences < 0 || sequences > 65535 || channels <= 0 || taps < 1 || taps > kMaxTaps || ldx < channels)
        return CIE_BAD_ARGUMENT;
    if (sequences == 0 || taps == 1) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid((channels + 255) / 256, sequences);
    if (dtype == CIE_F32)
        conv_keep_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(x), ldx, past, seq_slot, q_start_loc,
                                                     channels, taps);
    else if (dtype == CIE_BF16)
        conv_keep_kernel<bf16_t><<<grid, 256, 0, s>>>(static_cast<const bf16_t*>(x), ldx, past, seq_slot, q_start_loc,
                                                      channels, taps);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}

CIE_API int cie_gated_recurrence(void* stream, int dtype, const void* y_pre, long ldy, const void* x_in, long ldx,
                                 const void* u, const float* gates, int block_width, const float* rate, float* state,
                                 float* past, const int* seq_slot, const int* q_start_loc, void* out, int sequences,
                                 int channels, int taps, int segments) {
    if (sequences < 0 || sequences > 65535 || channels <= 0 || block_width <= 0 || channels % block_width || taps < 1 ||
        taps > kMaxTaps || ldy < channels || ldx < channels || segments < 1 || segments > kMaxSegments)
        return CIE_BAD_ARGUMENT;
    if (sequences == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
#define CIE_SCAN(T, CH)                                                                                             \
    gated_recurrence_kernel<T, CH><<<dim3((channels + CH - 1) / CH, sequences), CH * segments, 0, s>>>(               \
        static_cast<const T*>(y_pre), ldy, static_cast<const T*>(x_in), ldx, static_cast<const T*>(u), gates,          \
        block_width, rate, state, past, seq_slot, q_start_loc, static_cast<T*>(out), channels, taps, segments)
    if (dtype == CIE_F32 && segments == 1) CIE_SCAN(float, 64);
    else if (dtype == CIE_F32) CIE_SCAN(float, 16);
    else if (dtype == CIE_BF16 && segments == 1) CIE_SCAN(bf16_t, 64);
    else if (dtype == CIE_BF16) CIE_SCAN(bf16_t, 16);
#undef CIE_SCAN
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}
