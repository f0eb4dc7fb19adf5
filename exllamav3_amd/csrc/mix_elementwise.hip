// Row-wise kernels over a float32 residual stream: embedding, RMS norm, gated residual (+ the next norm), PolyNorm, the router's
// top-k softmax.  One workgroup per row; every reduction is float32.
#include "mix_common.cuh"

static thread_local char g_mix_err[512] = "";
void mix_set_error(const char* fmt, ...)
{
    va_list ap; va_start(ap, fmt); vsnprintf(g_mix_err, sizeof(g_mix_err), fmt, ap); va_end(ap);
}
int mix_check_launch(const char* what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { mix_set_error("%s: launch failed: %s", what, hipGetErrorString(e)); return EXL3_MIX_ERR_HIP; }
    return EXL3_MIX_OK;
}
extern "C" const char* exl3_mix_last_error(void) { return g_mix_err; }
extern "C" int exl3_mix_abi_version(void) { return EXL3_MIX_ABI_VERSION; }

#define ROW_THREADS 256
#define ROW_WAVES 4

template <typename T>
__global__ __launch_bounds__(ROW_THREADS) void embed_kernel(float* __restrict__ x, T* __restrict__ h, const T* __restrict__ table,
                                                            const int32_t* __restrict__ tokens, float scale, const float* __restrict__ norm_w,
                                                            float eps, int width, int vocab)
{
    __shared__ float red[ROW_WAVES];
    const int n = blockIdx.x;
    int tok = tokens[n];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    const T* src = table + (int64_t) tok * width;
    float* xr = x + (int64_t) n * width;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += ROW_THREADS)
    {
        float v = to_f(src[i]) * scale;
        xr[i] = v;
        ss += v * v;
    }
    if (!norm_w) return;
    ss = block_sum<ROW_WAVES>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float) width + eps);
    T* hr = h + (int64_t) n * width;
    for (int i = threadIdx.x; i < width; i += ROW_THREADS) hr[i] = from_f<T>(xr[i] * inv * norm_w[i]);
}

template <typename T>
__global__ __launch_bounds__(ROW_THREADS) void rms_norm_rows_kernel(T* __restrict__ h, const float* __restrict__ x, const int32_t* __restrict__ rows,
                                                                    const float* __restrict__ w, float eps, int width)
{
    __shared__ float red[ROW_WAVES];
    const int n = blockIdx.x;
    const float* xr = x + (int64_t) (rows ? rows[n] : n) * width;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += ROW_THREADS) { float v = xr[i]; ss += v * v; }
    ss = block_sum<ROW_WAVES>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float) width + eps);
    T* hr = h + (int64_t) n * width;
    for (int i = threadIdx.x; i < width; i += ROW_THREADS) hr[i] = from_f<T>(xr[i] * inv * w[i]);
}

template <typename T>
__global__ __launch_bounds__(ROW_THREADS) void gated_residual_kernel(float* __restrict__ x, const T* __restrict__ y, int64_t y_ld, const T* __restrict__ r,
                                                                     int64_t r_ld, const float* __restrict__ norm_w, T* __restrict__ h, float eps, int width)
{
    __shared__ float red[ROW_WAVES];
    const int n = blockIdx.x;
    float* xr = x + (int64_t) n * width;
    const T* yr = y + (int64_t) n * y_ld;
    const T* rr = r + (int64_t) n * r_ld;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += ROW_THREADS)
    {
        float v = xr[i] + to_f(yr[i]) * sigmoid_f(to_f(rr[i]));
        xr[i] = v;
        ss += v * v;
    }
    if (!norm_w) return;
    ss = block_sum<ROW_WAVES>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float) width + eps);
    T* hr = h + (int64_t) n * width;
    for (int i = threadIdx.x; i < width; i += ROW_THREADS) hr[i] = from_f<T>(xr[i] * inv * norm_w[i]);
}

template <typename T>
__global__ __launch_bounds__(ROW_THREADS) void polynorm_kernel(T* __restrict__ out, const T* __restrict__ z, int64_t z_ld, const float* __restrict__ coef,
                                                               float eps, int ff)
{
    __shared__ float red[3][ROW_WAVES];
    const int n = blockIdx.x;
    const T* zr = z + (int64_t) n * z_ld;
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (int i = threadIdx.x; i < ff; i += ROW_THREADS)
    {
        float v = to_f(zr[i]), v2 = v * v, v3 = v2 * v;
        s1 += v2; s2 += v2 * v2; s3 += v3 * v3;
    }
    s1 = wave_sum(s1); s2 = wave_sum(s2); s3 = wave_sum(s3);
    if ((threadIdx.x & 63) == 0) { red[0][threadIdx.x >> 6] = s1; red[1][threadIdx.x >> 6] = s2; red[2][threadIdx.x >> 6] = s3; }
    __syncthreads();
    s1 = s2 = s3 = 0.f;
    #pragma unroll
    for (int i = 0; i < ROW_WAVES; ++i) { s1 += red[0][i]; s2 += red[1][i]; s3 += red[2][i]; }
    const float i1 = 1.0f / sqrtf(s1 / (float) ff + eps), i2 = 1.0f / sqrtf(s2 / (float) ff + eps), i3 = 1.0f / sqrtf(s3 / (float) ff + eps);
    const float a = coef[0], b = coef[1], c = coef[2], e = coef[3];
    T* o = out + (int64_t) n * ff;
    for (int i = threadIdx.x; i < ff; i += ROW_THREADS)
    {
        float v = to_f(zr[i]), v2 = v * v;
        o[i] = from_f<T>(a * (v * i1) + b * (v2 * i2) + c * (v2 * v * i3) + e);
    }
}

__global__ void topk_softmax_kernel(int32_t* __restrict__ idx, float* __restrict__ wts, const float* __restrict__ logits, int n, int experts, int top)
{
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n) return;
    const float* l = logits + (int64_t) t * experts;
    int32_t* id = idx + (int64_t) t * top;
    float* w = wts + (int64_t) t * top;
    for (int r = 0; r < top; ++r)
    {
        int best = -1; float bv = 0.f;
        for (int e = 0; e < experts; ++e)
        {
            bool taken = false;
            for (int p = 0; p < r; ++p) taken |= (id[p] == e);
            if (taken) continue;
            float v = l[e];
            if (best < 0 || v > bv) { best = e; bv = v; }
        }
        id[r] = best; w[r] = bv;
    }
    const float m = w[0];
    float s = 0.f;
    for (int r = 0; r < top; ++r) { float e = expf(w[r] - m); w[r] = e; s += e; }
    for (int r = 0; r < top; ++r) w[r] = w[r] / s;
}

extern "C" int exl3_mix_embed(float* x, void* h, const void* table, const int32_t* tokens, float scale, const float* norm_w, float eps,
                              int n, int width, int vocab, int dtype, void* stream)
{
    MIX_CHECK(x && table && tokens && n >= 0 && width > 0 && vocab > 0 && (!norm_w || h), "mix_embed: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(embed_kernel<T>, dim3(n), dim3(ROW_THREADS), 0, (hipStream_t) stream, x, (T*) h, (const T*) table, tokens, scale,
                                             norm_w, eps, width, vocab));
    return mix_check_launch("mix_embed");
}

extern "C" int exl3_mix_rms_norm_rows(void* h, const float* x, const int32_t* rows, const float* w, float eps, int n, int width, int dtype, void* stream)
{
    MIX_CHECK(h && x && w && n >= 0 && width > 0, "mix_rms_norm_rows: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(rms_norm_rows_kernel<T>, dim3(n), dim3(ROW_THREADS), 0, (hipStream_t) stream, (T*) h, x, rows, w, eps, width));
    return mix_check_launch("mix_rms_norm_rows");
}

extern "C" int exl3_mix_gated_residual(float* x, const void* y, int64_t y_ld, const void* r, int64_t r_ld, const float* norm_w, void* h, float eps,
                                       int n, int width, int dtype, void* stream)
{
    MIX_CHECK(x && y && r && n >= 0 && width > 0 && y_ld >= width && r_ld >= width && (!norm_w || h), "mix_gated_residual: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(gated_residual_kernel<T>, dim3(n), dim3(ROW_THREADS), 0, (hipStream_t) stream, x, (const T*) y, y_ld, (const T*) r, r_ld,
                                             norm_w, (T*) h, eps, width));
    return mix_check_launch("mix_gated_residual");
}

extern "C" int exl3_mix_polynorm(void* out, const void* z, int64_t z_ld, const float* coef, float eps, int n, int ff, int dtype, void* stream)
{
    MIX_CHECK(out && z && coef && n >= 0 && ff > 0 && z_ld >= ff, "mix_polynorm: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(polynorm_kernel<T>, dim3(n), dim3(ROW_THREADS), 0, (hipStream_t) stream, (T*) out, (const T*) z, z_ld, coef, eps, ff));
    return mix_check_launch("mix_polynorm");
}

extern "C" int exl3_mix_topk_softmax(int32_t* idx, float* wts, const float* logits, int n, int experts, int top, void* stream)
{
    MIX_CHECK(idx && wts && logits && n >= 0 && experts > 0 && top > 0 && top <= experts, "mix_topk_softmax: bad arguments (top %d of %d)", top, experts);
    if (n == 0) return EXL3_MIX_OK;
    hipLaunchKernelGGL(topk_softmax_kernel, dim3((n + 63) / 64), dim3(64), 0, (hipStream_t) stream, idx, wts, logits, n, experts, top);
    return mix_check_launch("mix_topk_softmax");
}
