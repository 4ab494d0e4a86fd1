// What stands around a sublayer whose OUTPUT is normed before it joins the residual stream:
//     x <- x + mult * rmsnorm(scale_a * a + scale_b * b) * w
// (b optional: two branches that read the same input and are mixed with fixed weights), the rounded
// copy of the new x that the next sublayer's products read, and a gated linear unit with clamped
// halves. Sums and the residual stream are float32.
#include "fw_common.h"
#include "fw_kernels.h"

__device__ __forceinline__ float sublayer_sigmoid(float g) {
    if (g >= 0.0f) return 1.0f / (1.0f + expf(-g));
    const float e = expf(g);
    return e / (1.0f + e);
}

// One workgroup per row. y = scale_a a (+ scale_b b) is formed once and kept in registers (rows of up
// to 256 * NORM_ADD_HELD channels) or formed again in the second pass (wider rows).
#define NORM_ADD_HELD 16
template <typename T>
__global__ __launch_bounds__(256) void norm_scale_add_kernel(
    float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ b, float scale_a, float scale_b,
    const float* __restrict__ weight, int one_centered, float eps, float mult, T* __restrict__ rounded, int hidden) {
    __shared__ float scratch[16];
    const size_t row0 = (size_t)blockIdx.x * hidden;
    const bool held_all = hidden <= 256 * NORM_ADD_HELD;
    float held[NORM_ADD_HELD], was[NORM_ADD_HELD], scale[NORM_ADD_HELD];
    float sum = 0.0f;
    if (held_all) {
        // everything the row needs is asked for at once: the old x and the weight travel with a and b
#pragma unroll
        for (int u = 0; u < NORM_ADD_HELD; ++u) {
            const int i = threadIdx.x + 256 * u;
            float y = 0.0f;
            was[u] = scale[u] = 0.0f;
            if (i < hidden) {
                y = scale_a * a[row0 + i];
                if (b) y = fmaf(scale_b, b[row0 + i], y);
                was[u] = x[row0 + i];
                scale[u] = weight[i];
            }
            held[u] = y;
            sum = fmaf(y, y, sum);
        }
    } else {
        for (int i = threadIdx.x; i < hidden; i += 256) {
            float y = scale_a * a[row0 + i];
            if (b) y = fmaf(scale_b, b[row0 + i], y);
            sum = fmaf(y, y, sum);
        }
    }
    sum = block_sum(sum, scratch);
    const float inv = 1.0f / sqrtf(sum / (float)hidden + eps);
    const float one = one_centered ? 1.0f : 0.0f;
    if (held_all) {
#pragma unroll
        for (int u = 0; u < NORM_ADD_HELD; ++u) {
            const int i = threadIdx.x + 256 * u;
            if (i < hidden) {
                const float updated = was[u] + mult * (held[u] * inv * (scale[u] + one));
                x[row0 + i] = updated;
                if (rounded) store_from_float(rounded, row0 + i, updated);
            }
        }
    } else {
        for (int i = threadIdx.x; i < hidden; i += 256) {
            float y = scale_a * a[row0 + i];
            if (b) y = fmaf(scale_b, b[row0 + i], y);
            const float updated = x[row0 + i] + mult * (y * inv * (weight[i] + one));
            x[row0 + i] = updated;
            if (rounded) store_from_float(rounded, row0 + i, updated);
        }
    }
}

extern "C" int fw_norm_scale_add(float* x, const float* a, const float* b, float scale_a, float scale_b, const float* weight,
                                 int one_centered, float eps, float mult, void* rounded, int rounded_dtype, int rows,
                                 int hidden, void* stream) {
    FW_REQUIRE(rows >= 0 && hidden > 0, "norm_scale_add: bad sizes rows=%d hidden=%d", rows, hidden);
    FW_REQUIRE(eps > 0.0f, "norm_scale_add: eps must be positive");
    FW_REQUIRE(x && a && weight, "norm_scale_add: x, a and the weight are needed");
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (!rounded || rounded_dtype == FW_F32)
        norm_scale_add_kernel<float><<<rows, 256, 0, s>>>(x, a, b, scale_a, scale_b, weight, one_centered, eps, mult, (float*)rounded, hidden);
    else if (rounded_dtype == FW_BF16)
        norm_scale_add_kernel<bf16_t><<<rows, 256, 0, s>>>(x, a, b, scale_a, scale_b, weight, one_centered, eps, mult, (bf16_t*)rounded, hidden);
    else
        FW_REQUIRE(false, "norm_scale_add: unknown dtype %d", rounded_dtype);
    FW_LAUNCH_CHECK("norm_scale_add");
    return 0;
}

// float32 rows rounded to the activation type
__global__ void round_rows_kernel(const float* __restrict__ x, bf16_t* __restrict__ out, long long count) {
    for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < count; i += (long long)gridDim.x * blockDim.x)
        out[i] = float_to_bf16(x[i]);
}

extern "C" int fw_round_rows(const float* x, void* out, long long count, void* stream) {
    FW_REQUIRE(count >= 0, "round_rows: negative count");
    if (count == 0) return 0;
    const int blocks = (int)((count + 255) / 256 < 4096 ? (count + 255) / 256 : 4096);
    round_rows_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>(x, (bf16_t*)out, count);
    FW_LAUNCH_CHECK("round_rows");
    return 0;
}

// Gated linear unit with clamped halves: g = min(gate, limit), u = clamp(up, -limit, limit),
// out = g * sigmoid(alpha * g) * (u + shift). gate_up [rows][2 I]: gate columns, then up columns.
template <typename TI, typename TO>
__global__ void clamped_glu_kernel(const TI* __restrict__ gate_up, TO* __restrict__ out, int intermediate, float limit,
                                   float alpha, float shift) {
    const int row = blockIdx.y;
    const TI* source = gate_up + (size_t)row * 2 * intermediate;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < intermediate; i += gridDim.x * blockDim.x) {
        const float g = fminf(load_as_float(source, i), limit);
        const float u = fminf(fmaxf(load_as_float(source, (size_t)intermediate + i), -limit), limit);
        store_from_float(out, (size_t)row * intermediate + i, g * sublayer_sigmoid(alpha * g) * (u + shift));
    }
}

extern "C" int fw_clamped_glu(const void* gate_up, int in_dtype, void* out, int out_dtype, int rows, int intermediate,
                              float limit, float alpha, float shift, void* stream) {
    FW_REQUIRE(rows >= 0 && rows <= 65535 * 16 && intermediate > 0, "clamped_glu: bad sizes rows=%d intermediate=%d", rows, intermediate);
    FW_REQUIRE(limit > 0.0f, "clamped_glu: the limit must be positive");
    if (rows == 0) return 0;
    int across = (intermediate + 255) / 256;
    if (across > 64) across = 64;
    hipStream_t s = (hipStream_t)stream;
    for (int row0 = 0; row0 < rows; row0 += 65535) {
        const int now = rows - row0 < 65535 ? rows - row0 : 65535;
        dim3 grid(across, now);
        const size_t in_at = (size_t)row0 * 2 * intermediate, out_at = (size_t)row0 * intermediate;
#define FW_GLU_LAUNCH(TI, TO) \
    clamped_glu_kernel<TI, TO><<<grid, 256, 0, s>>>((const TI*)gate_up + in_at, (TO*)out + out_at, intermediate, limit, alpha, shift)
        if (in_dtype == FW_F32 && out_dtype == FW_F32) FW_GLU_LAUNCH(float, float);
        else if (in_dtype == FW_F32 && out_dtype == FW_BF16) FW_GLU_LAUNCH(float, bf16_t);
        else if (in_dtype == FW_BF16 && out_dtype == FW_BF16) FW_GLU_LAUNCH(bf16_t, bf16_t);
        else FW_REQUIRE(false, "clamped_glu: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
#undef FW_GLU_LAUNCH
    }
    FW_LAUNCH_CHECK("clamped_glu");
    return 0;
}

// ---- a sublayer between two norms ---------------------------------------------------------------------
// What joins a sublayer whose output passes a norm of its own to the residual stream, and hands the
// stream to the next reader, in one pass over the row:
//     x <- x + norm_a(a) * w            (norm_a: RMS, or with `centered` the mean taken off first)
//     next_out = next(x)                (next_kind 0: nothing; 1: x rounded to next_dtype; 2: RMS norm
//                                        of x times next_weight; 3: the same with the mean taken off)
// A norm here is v / sqrt(mean(v^2) + eps), v the values or their deviations from the row's mean. One
// workgroup per row; a row of up to 256 * JOIN_HELD values stays in registers between the passes, a
// wider one is read again. Every sum is a function of the row alone.
#define JOIN_HELD 16
template <typename T, bool HELD>
__global__ __launch_bounds__(256) void norm_add_norm_kernel(
    float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ weight, int centered, float eps,
    int next_kind, const float* __restrict__ next_weight, float next_eps, T* __restrict__ next_out, int hidden) {
    __shared__ float scratch[16];
    const size_t row0 = (size_t)blockIdx.x * hidden;
    constexpr int N = HELD ? JOIN_HELD : 1;
    float held[N], was[N], scale[N];
    const float count = (float)hidden;
    float sum = 0.0f;
    if (HELD) {
#pragma unroll
        for (int u = 0; u < N; ++u) {
            const int i = threadIdx.x + 256 * u;
            const bool in = i < hidden;
            held[u] = in ? a[row0 + i] : 0.0f;
            was[u] = in ? x[row0 + i] : 0.0f;
            scale[u] = in ? weight[i] : 0.0f;
            sum += held[u];
        }
    } else {
        for (int i = threadIdx.x; i < hidden; i += 256) sum += a[row0 + i];
    }
    const float mean = centered ? block_sum(sum, scratch) / count : 0.0f;
    float squares = 0.0f;
    if (HELD) {
#pragma unroll
        for (int u = 0; u < N; ++u) {
            const float d = threadIdx.x + 256 * u < hidden ? held[u] - mean : 0.0f;
            squares = fmaf(d, d, squares);
        }
    } else {
        for (int i = threadIdx.x; i < hidden; i += 256) {
            const float d = a[row0 + i] - mean;
            squares = fmaf(d, d, squares);
        }
    }
    const float inv = 1.0f / sqrtf(block_sum(squares, scratch) / count + eps);
    float new_sum = 0.0f;
    if (HELD) {
#pragma unroll
        for (int u = 0; u < N; ++u) {
            const int i = threadIdx.x + 256 * u;
            if (i < hidden) {
                was[u] += (held[u] - mean) * inv * scale[u];
                x[row0 + i] = was[u];
                new_sum += was[u];
            }
        }
    } else {
        for (int i = threadIdx.x; i < hidden; i += 256) {
            const float updated = x[row0 + i] + (a[row0 + i] - mean) * inv * weight[i];
            x[row0 + i] = updated;          // read again below by the thread that wrote it
            new_sum += updated;
        }
    }
    if (next_kind == 0) return;
    if (next_kind == 1) {
        if (HELD) {
#pragma unroll
            for (int u = 0; u < N; ++u) {
                const int i = threadIdx.x + 256 * u;
                if (i < hidden) store_from_float(next_out, row0 + i, was[u]);
            }
        } else {
            for (int i = threadIdx.x; i < hidden; i += 256) store_from_float(next_out, row0 + i, x[row0 + i]);
        }
        return;
    }
    const float next_mean = next_kind == 3 ? block_sum(new_sum, scratch) / count : 0.0f;
    float next_squares = 0.0f;
    if (HELD) {
#pragma unroll
        for (int u = 0; u < N; ++u) {
            const float d = threadIdx.x + 256 * u < hidden ? was[u] - next_mean : 0.0f;
            next_squares = fmaf(d, d, next_squares);
        }
    } else {
        for (int i = threadIdx.x; i < hidden; i += 256) {
            const float d = x[row0 + i] - next_mean;
            next_squares = fmaf(d, d, next_squares);
        }
    }
    const float next_inv = 1.0f / sqrtf(block_sum(next_squares, scratch) / count + next_eps);
    if (HELD) {
#pragma unroll
        for (int u = 0; u < N; ++u) {
            const int i = threadIdx.x + 256 * u;
            if (i < hidden) store_from_float(next_out, row0 + i, (was[u] - next_mean) * next_inv * next_weight[i]);
        }
    } else {
        for (int i = threadIdx.x; i < hidden; i += 256)
            store_from_float(next_out, row0 + i, (x[row0 + i] - next_mean) * next_inv * next_weight[i]);
    }
}

extern "C" int fw_norm_add_norm(float* x, const float* a, const float* weight, int centered, float eps, int next_kind,
                                const float* next_weight, float next_eps, void* next_out, int next_dtype, int rows,
                                int hidden, void* stream) {
    FW_REQUIRE(rows >= 0 && hidden > 0, "norm_add_norm: bad sizes rows=%d hidden=%d", rows, hidden);
    FW_REQUIRE(eps > 0.0f, "norm_add_norm: eps must be positive");
    FW_REQUIRE(x && a && weight, "norm_add_norm: x, a and the weight are needed");
    FW_REQUIRE(next_kind >= 0 && next_kind <= 3, "norm_add_norm: unknown kind %d of what follows", next_kind);
    FW_REQUIRE(next_kind == 0 || next_out, "norm_add_norm: what follows has nowhere to go");
    FW_REQUIRE(next_kind < 2 || (next_weight && next_eps > 0.0f), "norm_add_norm: the norm that follows needs a weight and a positive eps");
    FW_REQUIRE(next_kind == 0 || next_dtype == FW_F32 || next_dtype == FW_BF16, "norm_add_norm: unknown dtype %d", next_dtype);
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const bool held = hidden <= 256 * JOIN_HELD;
#define FW_JOIN_LAUNCH(T, HELD)                                                                                             \
    norm_add_norm_kernel<T, HELD><<<rows, 256, 0, s>>>(x, a, weight, centered, eps, next_kind, next_weight, next_eps, \
                                                       (T*)next_out, hidden)
    if (next_kind == 0 || next_dtype == FW_F32) {
        if (held) FW_JOIN_LAUNCH(float, true);
        else FW_JOIN_LAUNCH(float, false);
    } else {
        if (held) FW_JOIN_LAUNCH(bf16_t, true);
        else FW_JOIN_LAUNCH(bf16_t, false);
    }
#undef FW_JOIN_LAUNCH
    FW_LAUNCH_CHECK("norm_add_norm");
    return 0;
}
