// The gated delta rule: a linear recurrence over a matrix state per head, with the short causal
// convolutions in front of it and the gated norm behind it. Everything here is float32.
//
// Per head, with state S [dim][vdim], a token brings a query q and key k (dim channels, unit vectors),
// a value v (vdim channels), a write strength beta and a decay g per key channel:
//     S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// so the read-out sees the token's own write. Columns of S (value channels) never meet: a column is
// owned by four lanes, each holding a quarter of its rows in registers, and the two sums over the
// key channels are reductions over those four lanes. A segment's tokens are walked in order; what a
// token brings is staged through LDS a chunk of tokens at a time.
//
// The state is stored transposed, [slot][head][vdim][dim], so that the quarter columns a wave holds
// are one contiguous piece of memory.
#include "fw_common.h"
#include "fw_kernels.h"

#define DELTA_CHUNK 16          // tokens staged in LDS at a time
#define DELTA_COLUMNS 64        // value channels per workgroup (256 threads: four lanes a column)

__device__ __forceinline__ float fw_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float fw_softplus(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

// ---- what the recurrence reads, from the projections -----------------------------------------------
// One wave per (row, vector). Vectors 0..G-1: query heads, G..2G-1: key heads (dim channels each,
// convolution, silu, then unit length; queries also times dim^-1/2); then H value heads (vdim
// channels, convolution and silu); then H decay vectors (dim channels, no convolution):
// g = exp(-exp(A_log[h]) * softplus(a + dt_bias)); lane 0 of a decay vector also forms beta.
// proj [rows][proj_stride]: columns 0.. hold q | k | v (the convolution's inputs), column beta_col + h
// the write strength before its sigmoid. state [slots][C][L-1]: the inputs of the L-1 tokens before
// the segment, oldest first. The state is read here and moved on by conv_state_kernel afterwards.
template <typename TI>
__global__ __launch_bounds__(64) void delta_prepare_kernel(
    const TI* __restrict__ proj, int proj_stride, int beta_col, const TI* __restrict__ a, const float* __restrict__ taps,
    const float* __restrict__ conv_state, const float* __restrict__ A_log, const float* __restrict__ dt_bias,
    const int32_t* __restrict__ row_seg, const int32_t* __restrict__ seg_row0, const int32_t* __restrict__ seg_slot,
    float* __restrict__ qkv_out, float* __restrict__ decay_out, float* __restrict__ beta_out, int heads, int kv_heads,
    int dim, int vdim, int taps_count) {
    const int row = blockIdx.x, vec = blockIdx.y, lane = threadIdx.x;
    const int conv_channels = 2 * kv_heads * dim + heads * vdim;
    if (vec >= 2 * kv_heads + heads) {      // a decay vector
        const int h = vec - 2 * kv_heads - heads;
        const float rate = expf(A_log[h]);
        for (int i = lane; i < dim; i += 64) {
            const int at = h * dim + i;
            decay_out[(size_t)row * heads * dim + at] = expf(-rate * fw_softplus(load_as_float(a, (size_t)row * heads * dim + at) + dt_bias[at]));
        }
        if (lane == 0) beta_out[(size_t)row * heads + h] = fw_sigmoid(load_as_float(proj, (size_t)row * proj_stride + beta_col + h));
        return;
    }
    const bool value = vec >= 2 * kv_heads;
    const int width = value ? vdim : dim;
    const int c0 = value ? 2 * kv_heads * dim + (vec - 2 * kv_heads) * vdim : vec * dim;
    const int seg = row_seg[row];
    const int first = seg_row0[seg];
    const float* before = conv_state + (size_t)seg_slot[seg] * conv_channels * (taps_count - 1);
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
#pragma unroll
    for (int part = 0; part < 4; ++part) {
        const int i = lane + 64 * part;
        if (i < width) qkv_out[(size_t)row * conv_channels + c0 + i] = kept[part] * factor;
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

extern "C" int fw_delta_prepare(const void* proj, int dtype, int proj_stride, int beta_col, const void* a, const float* taps,
                                float* conv_state, const float* A_log, const float* dt_bias, const int32_t* row_seg,
                                const int32_t* seg_row0, const int32_t* seg_slot, float* qkv_out, float* decay_out,
                                float* beta_out, int rows, int segments, int heads, int kv_heads, int dim, int vdim,
                                int taps_count, int slots, void* stream) {
    FW_REQUIRE(rows >= 0 && segments >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
               "delta_prepare: heads %d must be a positive multiple of kv heads %d", heads, kv_heads);
    FW_REQUIRE(dim > 0 && dim <= 256 && vdim > 0 && vdim <= 256, "delta_prepare: dim %d and vdim %d must lie in 1..256", dim, vdim);
    FW_REQUIRE(taps_count >= 1 && taps_count <= 17, "delta_prepare: %d taps outside 1..17", taps_count);
    FW_REQUIRE(slots > 0, "delta_prepare: no state slots");
    const int channels = 2 * kv_heads * dim + heads * vdim;
    FW_REQUIRE(proj_stride >= channels && beta_col >= 0 && beta_col + heads <= proj_stride,
               "delta_prepare: the projections' rows (%d wide) do not hold %d channels and %d strengths at %d", proj_stride, channels, heads, beta_col);
    FW_REQUIRE(rows <= 1 << 20 && segments <= 65535 && 2 * kv_heads + 2 * heads <= 65535, "delta_prepare: too many rows, segments or heads");
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(rows, 2 * kv_heads + 2 * heads);
    dim3 state_grid((channels + 127) / 128, segments);
    if (dtype == FW_F32) {
        delta_prepare_kernel<float><<<grid, 64, 0, s>>>((const float*)proj, proj_stride, beta_col, (const float*)a, taps, conv_state, A_log,
                                                        dt_bias, row_seg, seg_row0, seg_slot, qkv_out, decay_out, beta_out, heads,
                                                        kv_heads, dim, vdim, taps_count);
        if (taps_count > 1)
            conv_state_kernel<float><<<state_grid, 128, 0, s>>>((const float*)proj, proj_stride, conv_state, seg_row0, seg_slot, channels, taps_count);
    } else if (dtype == FW_BF16) {
        delta_prepare_kernel<bf16_t><<<grid, 64, 0, s>>>((const bf16_t*)proj, proj_stride, beta_col, (const bf16_t*)a, taps, conv_state, A_log,
                                                         dt_bias, row_seg, seg_row0, seg_slot, qkv_out, decay_out, beta_out, heads,
                                                         kv_heads, dim, vdim, taps_count);
        if (taps_count > 1)
            conv_state_kernel<bf16_t><<<state_grid, 128, 0, s>>>((const bf16_t*)proj, proj_stride, conv_state, seg_row0, seg_slot, channels, taps_count);
    } else {
        FW_REQUIRE(false, "delta_prepare: unknown dtype %d", dtype);
    }
    FW_LAUNCH_CHECK("delta_prepare");
    return 0;
}

// ---- the recurrence -----------------------------------------------------------------------------
// Workgroup (segment, head, block of 64 value channels); thread = 4 * column + quarter. RPT: rows of
// a column per thread; the column's rows quarter * RPT .. + RPT - 1 (rows from dim on hold zeros).
// LDS per staged token: q, k, g (4 * RPT each, zero filled past dim), then the block's 64 values,
// then beta.
template <int RPT>
__global__ __launch_bounds__(256) void gated_delta_rule_kernel(
    const float* __restrict__ qkv, const float* __restrict__ decay, const float* __restrict__ beta,
    float* __restrict__ state, float* __restrict__ out, const int32_t* __restrict__ seg_row0,
    const int32_t* __restrict__ seg_slot, int heads, int kv_heads, int dim, int vdim) {
    constexpr int DP = 4 * RPT;
    constexpr int TOKEN = 3 * DP + DELTA_COLUMNS + 4;
    __shared__ __attribute__((aligned(16))) float staged[DELTA_CHUNK * TOKEN];
    const int seg = blockIdx.x, head = blockIdx.y, block = blockIdx.z;
    const int kvh = head / (heads / kv_heads);
    const int column = block * DELTA_COLUMNS + threadIdx.x / 4, quarter = threadIdx.x % 4;
    const bool live = column < vdim;
    const int first = seg_row0[seg], count = seg_row0[seg + 1] - first;
    const int conv_channels = 2 * kv_heads * dim + heads * vdim;
    float* mine = state + (((size_t)seg_slot[seg] * heads + head) * vdim + (live ? column : 0)) * dim;
    float S[RPT];
#pragma unroll
    for (int t = 0; t < RPT; ++t) {
        const int i = quarter * RPT + t;
        S[t] = (live && i < dim) ? mine[i] : 0.0f;
    }
    for (int base = 0; base < count; base += DELTA_CHUNK) {
        const int tokens = count - base < DELTA_CHUNK ? count - base : DELTA_CHUNK;
        __syncthreads();
        for (int item = threadIdx.x; item < tokens * TOKEN; item += 256) {
            const int token = item / TOKEN, at = item % TOKEN;
            const size_t row = (size_t)first + base + token;
            float value = 0.0f;
            if (at < DP) {
                if (at < dim) value = qkv[row * conv_channels + kvh * dim + at];
            } else if (at < 2 * DP) {
                if (at - DP < dim) value = qkv[row * conv_channels + (kv_heads + kvh) * dim + (at - DP)];
            } else if (at < 3 * DP) {
                if (at - 2 * DP < dim) value = decay[(row * heads + head) * dim + (at - 2 * DP)];
            } else if (at < 3 * DP + DELTA_COLUMNS) {
                const int c = block * DELTA_COLUMNS + (at - 3 * DP);
                if (c < vdim) value = qkv[row * conv_channels + 2 * kv_heads * dim + head * vdim + c];
            } else if (at == 3 * DP + DELTA_COLUMNS) {
                value = beta[row * heads + head];
            }
            staged[item] = value;
        }
        __syncthreads();
        for (int token = 0; token < tokens; ++token) {
            const float* t0 = staged + token * TOKEN;
            const float* qs = t0 + quarter * RPT;
            const float* ks = t0 + DP + quarter * RPT;
            const float* gs = t0 + 2 * DP + quarter * RPT;
            const float v = t0[3 * DP + threadIdx.x / 4];
            const float b = t0[3 * DP + DELTA_COLUMNS];
            float seen = 0.0f;
#pragma unroll
            for (int t = 0; t < RPT; ++t) {
                S[t] *= gs[t];
                seen = fmaf(S[t], ks[t], seen);
            }
            seen += __shfl_xor(seen, 1, 64);
            seen += __shfl_xor(seen, 2, 64);
            const float u = b * (v - seen);
            float read = 0.0f;
#pragma unroll
            for (int t = 0; t < RPT; ++t) {
                S[t] = fmaf(ks[t], u, S[t]);
                read = fmaf(S[t], qs[t], read);
            }
            read += __shfl_xor(read, 1, 64);
            read += __shfl_xor(read, 2, 64);
            if (live && quarter == 0) out[((size_t)first + base + token) * heads * vdim + head * vdim + column] = read;
        }
    }
    if (live) {
#pragma unroll
        for (int t = 0; t < RPT; ++t) {
            const int i = quarter * RPT + t;
            if (i < dim) mine[i] = S[t];
        }
    }
}

extern "C" int fw_gated_delta_rule(const float* qkv, const float* decay, const float* beta, float* state, float* out,
                                   const int32_t* seg_row0, const int32_t* seg_slot, int rows, int segments, int heads,
                                   int kv_heads, int dim, int vdim, int slots, void* stream) {
    FW_REQUIRE(rows >= 0 && segments >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
               "gated_delta_rule: heads %d must be a positive multiple of kv heads %d", heads, kv_heads);
    FW_REQUIRE(dim > 0 && dim <= 256 && vdim > 0, "gated_delta_rule: dim %d must lie in 1..256 and vdim %d be positive", dim, vdim);
    FW_REQUIRE(slots > 0 && segments <= 65535 && heads <= 65535, "gated_delta_rule: too many segments or heads, or no slots");
    if (rows == 0 || segments == 0) return 0;
    dim3 grid(segments, heads, (vdim + DELTA_COLUMNS - 1) / DELTA_COLUMNS);
    hipStream_t s = (hipStream_t)stream;
#define FW_DELTA_LAUNCH(RPT) \
    gated_delta_rule_kernel<RPT><<<grid, 256, 0, s>>>(qkv, decay, beta, state, out, seg_row0, seg_slot, heads, kv_heads, dim, vdim)
    if (dim <= 16) FW_DELTA_LAUNCH(4);
    else if (dim <= 32) FW_DELTA_LAUNCH(8);
    else if (dim <= 64) FW_DELTA_LAUNCH(16);
    else if (dim <= 128) FW_DELTA_LAUNCH(32);
    else FW_DELTA_LAUNCH(64);
#undef FW_DELTA_LAUNCH
    FW_LAUNCH_CHECK("gated_delta_rule");
    return 0;
}

// ---- behind the recurrence: per-head RMS norm, a weight, a sigmoid gate ------------------------------
// out[r][h][j] = o[r][h][j] * rsqrt(mean_j o^2 + eps) * weight[j] * sigmoid(gate[r][gate_col + h vdim + j])
template <typename TG, typename T>
__global__ __launch_bounds__(64) void gated_head_norm_kernel(const float* __restrict__ o, const TG* __restrict__ gate, int gate_stride,
                                                            const float* __restrict__ weight, T* __restrict__ out,
                                                            int heads, int vdim, float eps) {
    const int row = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const float* source = o + ((size_t)row * heads + head) * vdim;
    float sum = 0.0f;
    for (int j = lane; j < vdim; j += 64) sum += source[j] * source[j];
    sum = wave_sum(sum);
    const float inv = 1.0f / sqrtf(sum / (float)vdim + eps);
    for (int j = lane; j < vdim; j += 64) {
        const float g = fw_sigmoid(load_as_float(gate, (size_t)row * gate_stride + head * vdim + j));
        store_from_float(out, ((size_t)row * heads + head) * vdim + j, source[j] * inv * weight[j] * g);
    }
}

extern "C" int fw_gated_head_norm(const float* o, const void* gate, int gate_dtype, int gate_stride, const float* weight,
                                  void* out, int out_dtype, int rows, int heads, int vdim, float eps, void* stream) {
    FW_REQUIRE(rows >= 0 && heads > 0 && heads <= 65535 && vdim > 0, "gated_head_norm: bad sizes rows=%d heads=%d vdim=%d", rows, heads, vdim);
    FW_REQUIRE(gate_stride >= heads * vdim, "gated_head_norm: the gates' rows (%d wide) do not hold %d x %d", gate_stride, heads, vdim);
    if (rows == 0) return 0;
    dim3 grid(rows, heads);
    hipStream_t s = (hipStream_t)stream;
#define FW_GHN_LAUNCH(TG, T) \
    gated_head_norm_kernel<TG, T><<<grid, 64, 0, s>>>(o, (const TG*)gate, gate_stride, weight, (T*)out, heads, vdim, eps)
    if (gate_dtype == FW_F32 && out_dtype == FW_F32) FW_GHN_LAUNCH(float, float);
    else if (gate_dtype == FW_F32 && out_dtype == FW_BF16) FW_GHN_LAUNCH(float, bf16_t);
    else if (gate_dtype == FW_BF16 && out_dtype == FW_BF16) FW_GHN_LAUNCH(bf16_t, bf16_t);
    else FW_REQUIRE(false, "gated_head_norm: unsupported dtypes gate=%d out=%d", gate_dtype, out_dtype);
#undef FW_GHN_LAUNCH
    FW_LAUNCH_CHECK("gated_head_norm");
    return 0;
}
