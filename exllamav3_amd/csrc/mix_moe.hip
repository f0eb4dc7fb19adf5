// Unquantized experts for a few rows (decode, short prompts, and the float32 path): one wave per output element streams the chosen
// expert's weight row.  Sums are float32.  Long bfloat16 prompts go through the grouped matrix-core kernel instead (mix_moe_mfma.hip).
#include "mix_common.cuh"

template <typename T>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(T* __restrict__ hid, const T* __restrict__ h, const T* __restrict__ wg, const T* __restrict__ wu,
                                                          const int32_t* __restrict__ idx, int experts, int ff, int width, int top)
{
    const int row = blockIdx.x;                              // n * top + r
    const int j = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (j >= ff) return;
    const int lane = threadIdx.x & 63;
    int e = idx[row];
    e = e < 0 ? 0 : (e >= experts ? experts - 1 : e);
    const T* x = h + (int64_t) (row / top) * width;
    const T* g = wg + ((int64_t) e * ff + j) * width;
    const T* u = wu + ((int64_t) e * ff + j) * width;
    float ag = 0.f, au = 0.f;
    for (int c = lane; c < width; c += 64) { const float xv = to_f(x[c]); ag += xv * to_f(g[c]); au += xv * to_f(u[c]); }
    ag = wave_sum(ag); au = wave_sum(au);
    // the two projections leave the matrix product in the activation type before the activation, like any other linear of the model
    if (lane == 0) hid[(int64_t) row * ff + j] = from_f<T>(silu_f(to_f(from_f<T>(ag))) * to_f(from_f<T>(au)));
}

template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(T* __restrict__ y, const T* __restrict__ hid, const T* __restrict__ wd, const int32_t* __restrict__ idx,
                                                       const float* __restrict__ wts, int experts, int ff, int width, int top)
{
    const int n = blockIdx.x;
    const int col = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (col >= width) return;
    const int lane = threadIdx.x & 63;
    float acc = 0.f;
    for (int r = 0; r < top; ++r)
    {
        int e = idx[(int64_t) n * top + r];
        e = e < 0 ? 0 : (e >= experts ? experts - 1 : e);
        const T* hr = hid + ((int64_t) n * top + r) * ff;
        const T* wr = wd + ((int64_t) e * width + col) * ff;
        float a = 0.f;
        for (int c = lane; c < ff; c += 64) a += to_f(hr[c]) * to_f(wr[c]);
        acc += wts[(int64_t) n * top + r] * wave_sum(a);
    }
    if (lane == 0) y[(int64_t) n * width + col] = from_f<T>(acc);
}

extern "C" int exl3_mix_moe_gate_up(void* hid, const void* h, const void* wg, const void* wu, const int32_t* idx, int n, int top, int experts, int ff, int width,
                                    int dtype, void* stream)
{
    MIX_CHECK(hid && h && wg && wu && idx && n >= 0 && top > 0 && experts > 0 && ff > 0 && width > 0, "mix_moe_gate_up: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(moe_gate_up_kernel<T>, dim3(n * top, (ff + 3) / 4), dim3(256), 0, (hipStream_t) stream, (T*) hid, (const T*) h,
                                             (const T*) wg, (const T*) wu, idx, experts, ff, width, top));
    return mix_check_launch("mix_moe_gate_up");
}

extern "C" int exl3_mix_moe_down(void* y, const void* hid, const void* wd, const int32_t* idx, const float* wts, int n, int top, int experts, int ff, int width,
                                 int dtype, void* stream)
{
    MIX_CHECK(y && hid && wd && idx && wts && n >= 0 && top > 0 && experts > 0 && ff > 0 && width > 0, "mix_moe_down: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(moe_down_kernel<T>, dim3(n, (width + 3) / 4), dim3(256), 0, (hipStream_t) stream, (T*) y, (const T*) hid, (const T*) wd,
                                             idx, wts, experts, ff, width, top));
    return mix_check_launch("mix_moe_down");
}
