// Fused residual-add + RMSNorm.
//
//   x   = residual[row] (+ branch[row])        float32
//   var = mean(x^2);  y = x * (1 / sqrt(var + eps)) * weight
//
// The statistics, the scaling and the residual sum are float32; the output is
// rounded once to the activation type.  With `rows` given, only those rows are
// normalised (the rows whose logits are wanted) and the residual is not written
// back.  One workgroup per output row; the row is staged in LDS, so hidden*4
// bytes must fit in 64 KB.
#include "common.h"

template <typename T, typename W>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const T* __restrict__ branch,
                                   const W* __restrict__ weight, T* __restrict__ out,
                                   const int* __restrict__ rows, int hidden, float eps,
                                   int write_residual) {
    extern __shared__ float staged[];
    __shared__ float scratch[16];
    const int out_row = blockIdx.x;
    const int row = rows ? rows[out_row] : out_row;
    float* res = residual + static_cast<size_t>(row) * hidden;
    const T* add = branch ? branch + static_cast<size_t>(row) * hidden : nullptr;
    float sum_sq = 0.f;
    for (int h = threadIdx.x; h < hidden; h += blockDim.x) {
        float x = res[h];
        if (add) {
            x += to_float(add[h]);
            if (write_residual) res[h] = x;
        }
        staged[h] = x;
        sum_sq += x * x;
    }
    const float total = block_sum(sum_sq, scratch);
    const float inv = 1.0f / sqrtf(total / static_cast<float>(hidden) + eps);
    T* dst = out + static_cast<size_t>(out_row) * hidden;
    for (int h = threadIdx.x; h < hidden; h += blockDim.x)
        dst[h] = from_float<T>((staged[h] * inv) * to_float(weight[h]));
}

// bf16 activations and weight, hidden a multiple of 8: eight elements per thread, 16-byte accesses.
__global__ void add_rmsnorm_vec8_kernel(float* __restrict__ residual, const bf16_t* __restrict__ branch,
                                        const bf16_t* __restrict__ weight, bf16_t* __restrict__ out,
                                        int hidden, float eps) {
    extern __shared__ float staged[];
    __shared__ float scratch[16];
    const int row = blockIdx.x;
    float* res = residual + static_cast<size_t>(row) * hidden;
    const bf16_t* add = branch ? branch + static_cast<size_t>(row) * hidden : nullptr;
    float sum_sq = 0.f;
    for (int h = threadIdx.x * 8; h < hidden; h += blockDim.x * 8) {
        float4 x0 = *reinterpret_cast<const float4*>(res + h);
        float4 x1 = *reinterpret_cast<const float4*>(res + h + 4);
        if (add) {
            const uint4 raw = *reinterpret_cast<const uint4*>(add + h);
            x0.x += __uint_as_float(raw.x << 16); x0.y += __uint_as_float(raw.x & 0xffff0000u);
            x0.z += __uint_as_float(raw.y << 16); x0.w += __uint_as_float(raw.y & 0xffff0000u);
            x1.x += __uint_as_float(raw.z << 16); x1.y += __uint_as_float(raw.z & 0xffff0000u);
            x1.z += __uint_as_float(raw.w << 16); x1.w += __uint_as_float(raw.w & 0xffff0000u);
            *reinterpret_cast<float4*>(res + h) = x0;
            *reinterpret_cast<float4*>(res + h + 4) = x1;
        }
        *reinterpret_cast<float4*>(staged + h) = x0;
        *reinterpret_cast<float4*>(staged + h + 4) = x1;
        sum_sq += (x0.x * x0.x + x0.y * x0.y) + (x0.z * x0.z + x0.w * x0.w) + (x1.x * x1.x + x1.y * x1.y) +
                  (x1.z * x1.z + x1.w * x1.w);
    }
    const float total = block_sum(sum_sq, scratch);
    const float inv = 1.0f / sqrtf(total / static_cast<float>(hidden) + eps);
    bf16_t* dst = out + static_cast<size_t>(row) * hidden;
    for (int h = threadIdx.x * 8; h < hidden; h += blockDim.x * 8) {
        const float4 x0 = *reinterpret_cast<const float4*>(staged + h);
        const float4 x1 = *reinterpret_cast<const float4*>(staged + h + 4);
        const uint4 raw = *reinterpret_cast<const uint4*>(weight + h);
        uint4 packed;
        packed.x = pack_bf16((x0.x * inv) * __uint_as_float(raw.x << 16), (x0.y * inv) * __uint_as_float(raw.x & 0xffff0000u));
        packed.y = pack_bf16((x0.z * inv) * __uint_as_float(raw.y << 16), (x0.w * inv) * __uint_as_float(raw.y & 0xffff0000u));
        packed.z = pack_bf16((x1.x * inv) * __uint_as_float(raw.z << 16), (x1.y * inv) * __uint_as_float(raw.z & 0xffff0000u));
        packed.w = pack_bf16((x1.z * inv) * __uint_as_float(raw.w << 16), (x1.w * inv) * __uint_as_float(raw.w & 0xffff0000u));
        *reinterpret_cast<uint4*>(dst + h) = packed;
    }
}

template <typename T, typename W>
static int launch_norm(hipStream_t s, float* residual, const void* branch, const void* weight,
                       void* out, const int* rows, int n_out, int hidden, float eps,
                       int write_residual) {
    add_rmsnorm_kernel<T, W><<<n_out, n_out <= 64 ? 1024 : 256, hidden * sizeof(float), s>>>(
        residual, static_cast<const T*>(branch), static_cast<const W*>(weight), static_cast<T*>(out),
        rows, hidden, eps, write_residual);
    return cie_after_launch();
}

// RMSNorm of rows whose partial sums of squares are already known (left by the product that wrote the
// residual): no reduction over the row is needed, so a row is spread over several workgroups.
template <typename T, typename W>
__global__ void __launch_bounds__(256)
rmsnorm_from_sumsq_kernel(const float* __restrict__ residual, const float* __restrict__ sumsq, int parts,
                          const W* __restrict__ weight, T* __restrict__ out, int hidden, float eps) {
    __shared__ float scratch[16];
    const int row = blockIdx.y;
    float s = 0.f;
    for (int p = threadIdx.x; p < parts; p += blockDim.x) s += sumsq[static_cast<size_t>(row) * parts + p];
    const float inv = 1.0f / sqrtf(block_sum(s, scratch) / static_cast<float>(hidden) + eps);
    const int h = blockIdx.x * blockDim.x + threadIdx.x;
    if (h < hidden)
        out[static_cast<size_t>(row) * hidden + h] =
            from_float<T>((residual[static_cast<size_t>(row) * hidden + h] * inv) * to_float(weight[h]));
}

CIE_API int cie_rmsnorm_from_sumsq(void* stream, int wdtype, const float* residual, const float* sumsq, int parts,
                                   const void* weight, void* out, int rows, int hidden, float eps) {
    if (rows < 0 || rows > 65535 || hidden <= 0 || parts < 1 || !(eps > 0.f)) return CIE_BAD_ARGUMENT;
    if (rows == 0) return CIE_OK;
    dim3 grid((hidden + 255) / 256, rows);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (wdtype == CIE_BF16)
        rmsnorm_from_sumsq_kernel<bf16_t, bf16_t><<<grid, 256, 0, s>>>(
            residual, sumsq, parts, static_cast<const bf16_t*>(weight), static_cast<bf16_t*>(out), hidden, eps);
    else if (wdtype == CIE_F32)
        rmsnorm_from_sumsq_kernel<bf16_t, float><<<grid, 256, 0, s>>>(
            residual, sumsq, parts, static_cast<const float*>(weight), static_cast<bf16_t*>(out), hidden, eps);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}

// dtype: activation type of branch/out; wdtype: storage type of the weight.
CIE_API int cie_add_rmsnorm(void* stream, int dtype, int wdtype, float* residual, const void* branch,
                            const void* weight, void* out, const int* rows, int n_out, int hidden,
                            float eps, int write_residual) {
    if (n_out < 0 || hidden <= 0 || hidden * sizeof(float) > 64 * 1024 || !(eps > 0.f))
        return CIE_BAD_ARGUMENT;
    if (rows && write_residual) return CIE_BAD_ARGUMENT;
    if (n_out == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == CIE_F32 && wdtype == CIE_F32)
        return launch_norm<float, float>(s, residual, branch, weight, out, rows, n_out, hidden, eps, write_residual);
    if (dtype == CIE_BF16 && wdtype == CIE_BF16 && !rows && write_residual && hidden % 8 == 0) {
        add_rmsnorm_vec8_kernel<<<n_out, n_out <= 64 ? 1024 : 256, hidden * sizeof(float), s>>>(
            residual, static_cast<const bf16_t*>(branch), static_cast<const bf16_t*>(weight), static_cast<bf16_t*>(out),
            hidden, eps);
        return cie_after_launch();
    }
    if (dtype == CIE_BF16 && wdtype == CIE_BF16)
        return launch_norm<bf16_t, bf16_t>(s, residual, branch, weight, out, rows, n_out, hidden, eps, write_residual);
    if (dtype == CIE_BF16 && wdtype == CIE_F32)
        return launch_norm<bf16_t, float>(s, residual, branch, weight, out, rows, n_out, hidden, eps, write_residual);
    return CIE_BAD_ARGUMENT;
}

// Norm on a branch's output, then the add:
//   y = scale_a * branch[row] * sigmoid(branch_gate[row]) + scale_b * branch2[row]
//       + sum_p part_weight[row, p] * parts[row, p, :]           (float32 rows [tokens, parts, hidden], in order)
//   residual[row] += y / sqrt(mean(y^2) + eps) * weight
// Every addend but one may be absent (no gate: 1; no part weights: 1).  The weight comes as it multiplies: a weight
// stored around zero with the one added, a norm's weight times a scale per channel as their product.  With
// `rows_out` the new stream is also written in the activation type, for the products of a sublayer that reads the
// stream itself; with `next_weight` the RMS norm of the new stream under that weight is written to `normed_out`, for
// the sublayer that reads a norm of it.  Statistics, scaling and the sums are float32.  One workgroup per row, the
// row staged in LDS.
template <typename B, typename T>
__global__ void branch_norm_add_kernel(float* __restrict__ residual, const B* __restrict__ branch,
                                       const float* __restrict__ branch_gate, int gate_stride,
                                       const B* __restrict__ branch2, float scale_a, float scale_b,
                                       const float* __restrict__ parts, const float* __restrict__ part_weight, int n_parts,
                                       const float* __restrict__ weight, T* __restrict__ rows_out, int hidden,
                                       float eps, const float* __restrict__ next_weight, T* __restrict__ normed_out) {
    extern __shared__ float staged[];
    __shared__ float scratch[16];
    const size_t row = blockIdx.x;
    const B* add = branch ? branch + row * hidden : nullptr;
    const B* add2 = branch2 ? branch2 + row * hidden : nullptr;
    const float open = (branch && branch_gate) ? scale_a / (1.0f + expf(-branch_gate[row * gate_stride])) : scale_a;
    const float* extra = parts ? parts + row * n_parts * hidden : nullptr;
    const float* extra_w = (parts && part_weight) ? part_weight + row * n_parts : nullptr;
    float sum_sq = 0.f;
    for (int h = threadIdx.x; h < hidden; h += blockDim.x) {
        float y = add ? to_float(add[h]) * open : 0.f;
        if (add2) y = fmaf(scale_b, to_float(add2[h]), y);
        for (int p = 0; p < n_parts; ++p)
            y = fmaf(extra_w ? extra_w[p] : 1.0f, extra[static_cast<size_t>(p) * hidden + h], y);
        staged[h] = y;
        sum_sq += y * y;
    }
    const float total = block_sum(sum_sq, scratch);
    const float inv = 1.0f / sqrtf(total / static_cast<float>(hidden) + eps);
    float* res = residual + row * hidden;
    T* dst = rows_out ? rows_out + row * hidden : nullptr;
    float next_sq = 0.f;
    for (int h = threadIdx.x; h < hidden; h += blockDim.x) {
        const float x = res[h] + (staged[h] * inv) * weight[h];
        res[h] = x;
        if (dst) dst[h] = from_float<T>(x);
        staged[h] = x;
        next_sq += x * x;
    }
    if (!next_weight) return;
    const float next_total = block_sum(next_sq, scratch);
    const float next_inv = 1.0f / sqrtf(next_total / static_cast<float>(hidden) + eps);
    T* normed = normed_out + row * hidden;
    for (int h = threadIdx.x; h < hidden; h += blockDim.x)
        normed[h] = from_float<T>((staged[h] * next_inv) * next_weight[h]);
}

// bdtype: storage type of `branch` and `branch2` (ignored without them); dtype: type of rows_out and normed_out.
CIE_API int cie_branch_norm_add(void* stream, int bdtype, int dtype, float* residual, const void* branch,
                                const float* branch_gate, int gate_stride, const void* branch2, float scale_a,
                                float scale_b, const float* parts, const float* part_weight, int n_parts,
                                const float* weight, void* rows_out, int tokens, int hidden, float eps,
                                const float* next_weight, void* normed_out) {
    if (tokens < 0 || hidden <= 0 || hidden * sizeof(float) > 64 * 1024 || !(eps > 0.f) || n_parts < 0 ||
        (n_parts > 0 && !parts) || (!branch && !branch2 && n_parts == 0) || gate_stride < 1 ||
        (next_weight && !normed_out))
        return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int threads = tokens <= 64 ? 1024 : 256;
    const size_t lds = hidden * sizeof(float);
    if (!parts) n_parts = 0;
    const bool any = branch || branch2;
#define CIE_BRANCH_NORM(B, T)                                                                                        \
    branch_norm_add_kernel<B, T><<<tokens, threads, lds, s>>>(                                                          \
        residual, static_cast<const B*>(branch), branch_gate, gate_stride, static_cast<const B*>(branch2), scale_a,       \
        scale_b, parts, part_weight, n_parts, weight, static_cast<T*>(rows_out), hidden, eps, next_weight,                \
        static_cast<T*>(normed_out))
    if (dtype == CIE_F32 && (bdtype == CIE_F32 || !any)) CIE_BRANCH_NORM(float, float);
    else if (dtype == CIE_BF16 && bdtype == CIE_BF16) CIE_BRANCH_NORM(bf16_t, bf16_t);
    else if (dtype == CIE_BF16 && (bdtype == CIE_F32 || !any)) CIE_BRANCH_NORM(float, bf16_t);
#undef CIE_BRANCH_NORM
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}

// ---------------------------------------------------------------------------------------------- norm in groups
// The residual add of a layer that norms what its sublayers read, with everything a branch can still owe the stream,
// and an RMS norm whose statistics run over equal consecutive parts of the row:
//
//   x = residual[row] + branch[row] * sigmoid(branch_gate[row])            (branch; the gate one logit per row, rows
//                                                                           `gate_stride` floats apart)
//                     + sum_p part_weight[row, p] * parts[row, p, :]       (float32 rows still to be summed, in order)
//                     + plus[row]                                          (float32 rows, e.g. the embedding's again)
//   y[g] = x[g] / sqrt(mean(x[g]^2) + eps) * weight[g]                     for each of the `groups` parts g of the row
//
// Every addend may be absent.  Sums, statistics and scaling are float32; the row is staged in LDS.  With `rows`
// given only those rows are normed and the stream is not written back.  A wave takes the groups in turn, so the
// statistics need no barrier per group.
template <typename B, typename T>
__global__ void group_norm_add_kernel(float* __restrict__ residual, const B* __restrict__ branch,
                                      const float* __restrict__ branch_gate, int gate_stride,
                                      const float* __restrict__ parts, const float* __restrict__ part_weight, int n_parts,
                                      const float* __restrict__ plus, const float* __restrict__ weight,
                                      T* __restrict__ out, const int* __restrict__ rows, int hidden, int groups,
                                      float eps, int write_residual) {
    extern __shared__ float staged[];  // [hidden], then [groups]
    float* inverse = staged + hidden;
    const int out_row = blockIdx.x;
    const size_t row = rows ? rows[out_row] : out_row;
    float* res = residual + row * hidden;
    const B* add = branch ? branch + row * hidden : nullptr;
    const float open = (branch && branch_gate) ? 1.0f / (1.0f + expf(-branch_gate[row * gate_stride])) : 1.0f;
    const float* extra = n_parts > 0 ? parts + row * n_parts * hidden : nullptr;
    const float* extra_w = (n_parts > 0 && part_weight) ? part_weight + row * n_parts : nullptr;
    const float* more = plus ? plus + row * hidden : nullptr;
    for (int h = threadIdx.x; h < hidden; h += blockDim.x) {
        float x = res[h];
        if (add) x += to_float(add[h]) * open;
        for (int p = 0; p < n_parts; ++p)
            x += (extra_w ? extra_w[p] : 1.0f) * extra[static_cast<size_t>(p) * hidden + h];
        if (more) x += more[h];
        if (write_residual) res[h] = x;
        staged[h] = x;
    }
    __syncthreads();
    const int lane = threadIdx.x % kWave;
    const int waves = blockDim.x / kWave;
    const int per = hidden / groups;
    for (int g = threadIdx.x / kWave; g < groups; g += waves) {
        float sum_sq = 0.f;
        for (int h = lane; h < per; h += kWave) {
            const float x = staged[g * per + h];
            sum_sq += x * x;
        }
        sum_sq = wave_sum(sum_sq);
        if (lane == 0) inverse[g] = 1.0f / sqrtf(sum_sq / static_cast<float>(per) + eps);
    }
    __syncthreads();
    T* dst = out + static_cast<size_t>(out_row) * hidden;
    for (int h = threadIdx.x; h < hidden; h += blockDim.x)
        dst[h] = from_float<T>((staged[h] * inverse[h / per]) * weight[h]);
}

// bdtype: storage type of `branch` (ignored without one); dtype: type of `out`.  `weight` float32 [hidden].
CIE_API int cie_group_norm_add(void* stream, int bdtype, int dtype, float* residual, const void* branch,
                               const float* branch_gate, int gate_stride, const float* parts, const float* part_weight,
                               int n_parts, const float* plus, const float* weight, void* out, const int* rows, int n_rows,
                               int hidden, int groups, float eps) {
    if (n_rows < 0 || hidden <= 0 || groups <= 0 || hidden % groups || !(eps > 0.f) || n_parts < 0 || gate_stride < 1 ||
        (n_parts > 0 && !parts) || (static_cast<size_t>(hidden) + groups) * sizeof(float) > 64 * 1024 || !weight || !out)
        return CIE_BAD_ARGUMENT;
    if (n_rows == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int threads = n_rows <= 64 ? 1024 : 256;
    const size_t lds = (static_cast<size_t>(hidden) + groups) * sizeof(float);
    if (!parts) n_parts = 0;
    const int write_residual = (rows == nullptr && (branch || n_parts > 0 || plus)) ? 1 : 0;
    if (dtype == CIE_F32 && (bdtype == CIE_F32 || !branch))
        group_norm_add_kernel<float, float><<<n_rows, threads, lds, s>>>(
            residual, static_cast<const float*>(branch), branch_gate, gate_stride, parts, part_weight, n_parts, plus,
            weight,
            static_cast<float*>(out), rows, hidden, groups, eps, write_residual);
    else if (dtype == CIE_BF16 && (bdtype == CIE_BF16 || !branch))
        group_norm_add_kernel<bf16_t, bf16_t><<<n_rows, threads, lds, s>>>(
            residual, static_cast<const bf16_t*>(branch), branch_gate, gate_stride, parts, part_weight, n_parts, plus,
            weight,
            static_cast<bf16_t*>(out), rows, hidden, groups, eps, write_residual);
    else if (dtype == CIE_BF16 && bdtype == CIE_F32)
        group_norm_add_kernel<float, bf16_t><<<n_rows, threads, lds, s>>>(
            residual, static_cast<const float*>(branch), branch_gate, gate_stride, parts, part_weight, n_parts, plus,
            weight,
            static_cast<bf16_t*>(out), rows, hidden, groups, eps, write_residual);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}
