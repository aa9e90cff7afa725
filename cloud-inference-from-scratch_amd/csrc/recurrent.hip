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
// with zeros to `padded` numbers per head: [tokens, heads, 2, padded].  (b) The walk over the tokens, below.  (c) The
// head's norm and the gate, which need all value columns of a head.
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

// A barrier for what the waves of a workgroup hand each other through LDS.  It waits for the wave's LDS traffic only:
// loads from memory that are under way stay under way (`__syncthreads` waits for them too, which would put a block's
// way from memory in front of every barrier of a loop that fetches a block ahead).
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// (b') The same walk for sequences that bring many tokens (a prompt's portion), in blocks of 32 tokens on the matrix
// cores, float32 throughout (`v_mfma_f32_16x16x4_f32`: operands and sums are plain float32).  With S the memory in
// front of a block, i and j tokens of the block and f the head's decay:
//     o_i   = f^(i+1) * (S^T q_i)  +  sum_{j <= i} f^(i-j) (q_i . k_j) v_j
//     S_new = f^n * S  +  sum_j f^(n-1-j) k_j v_j^T          (n the block's tokens: 32, or fewer at the end)
// One workgroup of four waves takes (sequence, head, 16 value columns) and walks the blocks in order.  The block's
// queries, keys and values wait in LDS (fetched into registers a block ahead).  Wave w keeps rows of S in the matrix
// cores' result layout, where they serve as the second operand of S^T q as they are; it makes one 16 x 16 tile of
// q . k (the tile above the diagonal is zero), and its share of S^T q, of the block's own sum (tokens 8w .. 8w + 7)
// and of the new S; the waves' shares of o meet in LDS in the waves' order.  Powers of f come from a table made by
// repeated multiplication, as the walk token by token makes them.
typedef float acc4_t __attribute__((ext_vector_type(4)));
constexpr int kBlockTokens = 32;
constexpr int kBlockCols = 16;
constexpr int kScoreStride = kBlockTokens + 4;

// TPW: tiles of 16 rows of S that a wave keeps (the head's `padded` numbers are at most 64 * TPW)
template <typename T, int TPW>
__global__ void __launch_bounds__(256)
retention_blocks_kernel(const T* __restrict__ proj, long ldp, int v_off, const float* __restrict__ turned,
                        const float* __restrict__ decay, float* __restrict__ state, const int* __restrict__ seq_slot,
                        const int* __restrict__ q_start_loc, float* __restrict__ raw, int heads, int dim, int vdim,
                        int padded, int act) {
    extern __shared__ float4 lds4[];
    float* lds = reinterpret_cast<float*>(lds4);
    const int stride = padded + 4;                       // (a row's start moves on by four banks)
    float* q_s = lds;                                    // [32][stride]
    float* k_s = q_s + kBlockTokens * stride;            // [32][stride]
    float* v_s = k_s + kBlockTokens * stride;            // [32][16]
    float* p_s = v_s + kBlockTokens * kBlockCols;        // [32][36]: f^(i-j) (q_i . k_j), zero above the diagonal
    float* red = p_s + kBlockTokens * kScoreStride;      // [4][32][16]: the waves' shares of o
    float* pw = red + 4 * kBlockTokens * kBlockCols;     // [33]: powers of the decay
    const int seq = blockIdx.x / heads;
    const int head = blockIdx.x - seq * heads;
    const int v0 = blockIdx.y * kBlockCols;
    const int first = q_start_loc[seq];
    const int count = q_start_loc[seq + 1] - first;
    const int slot = seq_slot[seq];
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int l16 = lane % 16;
    const int g = lane / 16;
    const int tiles = padded / 16;
    const bool col_ok = v0 + l16 < vdim;
    if (threadIdx.x == 0) {
        float f = 1.0f;
        const float fade = decay[head];
        for (int n = 0; n <= kBlockTokens; ++n) {
            pw[n] = f;
            f *= fade;
        }
    }
    // rows of S: lane (g, l16), number r of tile t holds row 16 t + 4 g + r of column v0 + l16 (the result layout)
    float* mem = state + ((static_cast<size_t>(slot) * heads + head) * dim) * vdim + v0 + l16;
    acc4_t S[TPW];
#pragma unroll
    for (int u = 0; u < TPW; ++u)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = 16 * (wave * TPW + u) + 4 * g + r;
            S[u][r] = (col_ok && row < dim) ? mem[static_cast<size_t>(row) * vdim] : 0.f;
        }
    // which pieces of a block this thread fetches and where they go in LDS does not change from block to block
    // (divisions by sizes that only the launch knows: made once, not per block)
    const int pieces = padded / 2;                       // 16-byte pieces of one token's query and key
    int piece_token[4 * TPW], piece_from[4 * TPW], piece_to[4 * TPW];
#pragma unroll
    for (int i = 0; i < 4 * TPW; ++i) {
        const int idx = min(static_cast<int>(threadIdx.x) + i * 256, kBlockTokens * pieces - 1);
        const int t = idx / pieces;
        const int within = idx - t * pieces;
        const int side = within / (padded / 4);          // 0: the query, 1: the key
        piece_token[i] = t;
        piece_from[i] = within * 4;
        piece_to[i] = (side ? kBlockTokens * stride : 0) + t * stride + (within - side * (padded / 4)) * 4;
    }
    const T* values = proj + v_off + head * vdim;
    piece_t ahead[4 * TPW];
    T ahead_v[2];  // (as stored: a conversion right behind the load would wait for it, and for all loads before it)
#define CIE_BLOCKS_FETCH(from)                                                                                        \
    {                                                                                                                 \
        const int last = min(kBlockTokens, count - (from)) - 1;                                                       \
        const float* base = turned + (static_cast<size_t>(first + (from)) * heads + head) * 2 * padded;               \
        _Pragma("unroll") for (int i = 0; i < 4 * TPW; ++i)                                                           \
            ahead[i] = *reinterpret_cast<const piece_t*>(                                                             \
                base + static_cast<size_t>(min(piece_token[i], last)) * heads * 2 * padded + piece_from[i]);          \
        _Pragma("unroll") for (int i = 0; i < 2; ++i) {                                                               \
            const int idx = static_cast<int>(threadIdx.x) + i * 256;                                                  \
            const int t = min(idx / kBlockCols, last);                                                                \
            const int c = min(v0 + idx % kBlockCols, vdim - 1);                                                       \
            ahead_v[i] = values[static_cast<size_t>(first + (from) + t) * ldp + c];                                   \
        }                                                                                                             \
    }
    // the powers of the decay that this lane applies: they depend on its place, and on the block's length
    lds_barrier();                                       // (the table)
    const int ti = wave >> 1, tj = wave & 1;             // this wave's tile of the scores
    float p_fade[4], o_fade[2][4], k_fade[kBlockTokens / 4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int apart = 16 * (ti - tj) + 4 * g + r - l16;  // i - j
        p_fade[r] = apart >= 0 ? pw[min(apart, kBlockTokens)] : 0.f;
        o_fade[0][r] = pw[4 * g + r + 1];
        o_fade[1][r] = pw[16 + 4 * g + r + 1];
    }
    int faded_for = -1;
    float keep = 0.f;
    if (count > 0) CIE_BLOCKS_FETCH(0)
    for (int c0 = 0; c0 < count; c0 += kBlockTokens) {
        const int cn = min(kBlockTokens, count - c0);
        if (cn != faded_for) {                           // (the first block, and a last one that is shorter)
            faded_for = cn;
            keep = pw[cn];
#pragma unroll
            for (int kk = 0; kk < kBlockTokens / 4; ++kk) k_fade[kk] = pw[max(cn - 1 - (4 * kk + g), 0)];
        }
        // the block into LDS; rows past the block's last token are zero
#pragma unroll
        for (int i = 0; i < 4 * TPW; ++i)
            if (static_cast<int>(threadIdx.x) + i * 256 < kBlockTokens * pieces)
                *reinterpret_cast<piece_t*>(lds + piece_to[i]) =
                    piece_token[i] < cn ? ahead[i] : piece_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int idx = threadIdx.x + i * 256;
            v_s[idx] = (idx / kBlockCols < cn && v0 + idx % kBlockCols < vdim) ? activated(to_float(ahead_v[i]), act) : 0.f;
        }
        lds_barrier();
        if (c0 + kBlockTokens < count) CIE_BLOCKS_FETCH(c0 + kBlockTokens)
        // this wave's tile of the scores
        {
            acc4_t p = {0.f, 0.f, 0.f, 0.f};
            if (tj <= ti) {
                // (a lane reads four neighbouring numbers at once and spends them on four products: which four
                // numbers of the sum a product takes does not matter as long as both operands agree)
                const float* qa = q_s + (16 * ti + l16) * stride + 4 * g;
                const float* kb = k_s + (16 * tj + l16) * stride + 4 * g;
                acc4_t p1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int m = 0; m < 4 * TPW; ++m) {
                    if (m >= tiles) break;
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
            for (int r = 0; r < 4; ++r)
                p_s[(16 * ti + 4 * g + r) * kScoreStride + 16 * tj + l16] = p[r] * p_fade[r];
        }
        // this wave's share of S^T q, faded by the tokens' places in the block
        acc4_t o[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
        for (int u = 0; u < TPW; ++u) {
            const int t = wave * TPW + u;
            if (t < tiles) {
                const float4 a0 = *reinterpret_cast<const float4*>(q_s + l16 * stride + 16 * t + 4 * g);
                const float4 a1 = *reinterpret_cast<const float4*>(q_s + (16 + l16) * stride + 16 * t + 4 * g);
                o[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0.x, S[u][0], o[0], 0, 0, 0);
                o[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1.x, S[u][0], o[1], 0, 0, 0);
                o[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0.y, S[u][1], o[0], 0, 0, 0);
                o[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1.y, S[u][1], o[1], 0, 0, 0);
                o[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0.z, S[u][2], o[0], 0, 0, 0);
                o[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1.z, S[u][2], o[1], 0, 0, 0);
                o[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0.w, S[u][3], o[0], 0, 0, 0);
                o[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1.w, S[u][3], o[1], 0, 0, 0);
            }
        }
#pragma unroll
        for (int rt = 0; rt < 2; ++rt)
#pragma unroll
            for (int r = 0; r < 4; ++r) o[rt][r] *= o_fade[rt][r];
        lds_barrier();
        // ... of the block's own sum: tokens 8 w .. 8 w + 7
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            const int j = 8 * wave + 4 * kk + g;
            const float vb = v_s[j * kBlockCols + l16];
            o[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(p_s[l16 * kScoreStride + j], vb, o[0], 0, 0, 0);
            o[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(p_s[(16 + l16) * kScoreStride + j], vb, o[1], 0, 0, 0);
        }
#pragma unroll
        for (int rt = 0; rt < 2; ++rt)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                red[(wave * kBlockTokens + 16 * rt + 4 * g + r) * kBlockCols + l16] = o[rt][r];
        // ... and of the new S
        {
#pragma unroll
            for (int u = 0; u < TPW; ++u) {
                const int t = wave * TPW + u;
                if (t < tiles) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) S[u][r] *= keep;
#pragma unroll
                    for (int kk = 0; kk < kBlockTokens / 4; ++kk) {
                        const int j = 4 * kk + g;
                        const float ka = k_s[j * stride + 16 * t + l16] * k_fade[kk];
                        S[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(ka, v_s[j * kBlockCols + l16], S[u], 0, 0, 0);
                    }
                }
            }
        }
        lds_barrier();
        for (int idx = threadIdx.x; idx < cn * kBlockCols; idx += blockDim.x) {
            const int c = idx % kBlockCols;
            if (v0 + c >= vdim) continue;
            float sum = red[idx];
            for (int w = 1; w < 4; ++w) sum += red[w * kBlockTokens * kBlockCols + idx];
            raw[static_cast<size_t>(first + c0 + idx / kBlockCols) * heads * vdim + head * vdim + v0 + c] = sum;
        }
    }
#undef CIE_BLOCKS_FETCH
#pragma unroll
    for (int u = 0; u < TPW; ++u)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = 16 * (wave * TPW + u) + 4 * g + r;
            if (col_ok && row < dim) mem[static_cast<size_t>(row) * vdim] = S[u][r];
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
template <typename T>
__global__ void __launch_bounds__(256)
causal_conv_kernel(const T* __restrict__ x, long ldx, const T* __restrict__ taps_w, const T* __restrict__ bias,
                   const float* __restrict__ past, const int* __restrict__ seq_of_token, const int* __restrict__ seq_slot,
                   const int* __restrict__ q_start_loc, T* __restrict__ out, int channels, int taps) {
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
    out[static_cast<size_t>(token) * channels + c] = from_float<T>(acc);
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
                          int norm_span, const float* norm_weight, int gate_act, int blocks) {
    if (act < 0 || act > 1 || norm_span < 1 || heads % norm_span || gate_act < 0 || gate_act > 1) return CIE_BAD_ARGUMENT;
    if (blocks) {
        // the walk in blocks on the matrix cores: one plane of o, queries and keys padded to whole tiles of 16
        groups = 1;
        rows_per_thread = 16;
        parts = (dim + 15) / 16;
        slice = vdim < kBlockCols ? vdim : kBlockCols;
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
    const size_t blocks_lds = sizeof(float) * (2 * static_cast<size_t>(kBlockTokens) * (padded + 4) + kBlockTokens * kBlockCols +
                                               kBlockTokens * kScoreStride + 4 * kBlockTokens * kBlockCols + 36);
    const int value_slices = (vdim + kBlockCols - 1) / kBlockCols;
    if (blocks && (padded > 256 || blocks_lds > 64 * 1024 || value_slices > 65535 ||
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
        // (the workgroups of one head follow each other at a distance of `sequences * heads`: where that is a multiple
        // of eight they share an XCD, and its L2 holds the head's queries and keys for all of them)
        const dim3 block_grid(sequences * heads, value_slices);
#define CIE_BLOCKS(T, TPW)                                                                                            \
    retention_blocks_kernel<T, TPW><<<block_grid, 256, blocks_lds, s>>>(static_cast<const T*>(proj), ldp, v_off, turned,   \
                                                                          decay, state, seq_slot, q_start_loc, raw, heads, \
                                                                          dim, vdim, padded, act)
        if (dtype == CIE_F32) {
            if (padded <= 64) CIE_BLOCKS(float, 1);
            else if (padded <= 128) CIE_BLOCKS(float, 2);
            else CIE_BLOCKS(float, 4);
        } else {
            if (padded <= 64) CIE_BLOCKS(bf16_t, 1);
            else if (padded <= 128) CIE_BLOCKS(bf16_t, 2);
            else CIE_BLOCKS(bf16_t, 4);
        }
#undef CIE_BLOCKS
        code = cie_after_launch();
        parts = 1;
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
                            void* out, int tokens, int channels, int taps) {
    if (tokens < 0 || tokens > 65535 * 1 || channels <= 0 || taps < 1 || taps > kMaxTaps || ldx < channels) return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid((channels + 255) / 256, tokens);
    if (dtype == CIE_F32)
        causal_conv_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(x), ldx, static_cast<const float*>(taps_w),
                                                      static_cast<const float*>(bias), past, seq_of_token, seq_slot,
                                                      q_start_loc, static_cast<float*>(out), channels, taps);
    else if (dtype == CIE_BF16)
        causal_conv_kernel<bf16_t><<<grid, 256, 0, s>>>(static_cast<const bf16_t*>(x), ldx, static_cast<const bf16_t*>(taps_w),
                                                       static_cast<const bf16_t*>(bias), past, seq_of_token, seq_slot,
                                                       q_start_loc, static_cast<bf16_t*>(out), channels, taps);
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
