// Gated linear attention with a decay per key channel: the token-by-token form (decode, and the exact float32 prefill) and the
// output stage (per-head RMS norm, silu gate).  State, decays, logarithms and every product that enters the recurrence are float32.
//
// Work split of the scan: one workgroup of 4 waves per (sequence, head, block of 64 value columns).  Lane = value column; wave w
// owns the key channels w, w + 4, w + 8, ... (DR of them per lane, in registers).  A chunk of SCAN_TC (16 or 8) tokens is staged in LDS
// (q, k, alpha as float32; alpha computed here from the low-rank decay input), the waves run the recurrence over the chunk without
// a barrier, and the partial outputs of the four waves are added through LDS at the end of the chunk.
#include "mix_common.cuh"

#define SCAN_WAVES 4

template <typename T, int DR>
__global__ __launch_bounds__(256) void gla_scan_kernel(float* __restrict__ o, float* __restrict__ state, const T* __restrict__ q, int64_t q_ld,
                                                       const T* __restrict__ k, int64_t k_ld, const T* __restrict__ v, int64_t v_ld,
                                                       const T* __restrict__ lr, int64_t lr_ld, const T* __restrict__ a2, const float* __restrict__ a2_bias,
                                                       const int32_t* __restrict__ cu, const int32_t* __restrict__ slots, const int32_t* __restrict__ pos0,
                                                       int heads, int dim, int vdim, int rank, float inv_tau, float q_scale, int SCAN_TC)
{
    extern __shared__ float smem[];
    float* qs = smem;                                  // [SCAN_TC][dim]
    float* ks = qs + SCAN_TC * dim;
    float* as = ks + SCAN_TC * dim;
    float* vs = as + SCAN_TC * dim;                    // [SCAN_TC][64]
    float* part = vs + SCAN_TC * 64;                   // [SCAN_TC][SCAN_WAVES][64]
    const int b = blockIdx.x, h = blockIdx.y, vt = blockIdx.z;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int col = vt * 64 + lane;
    const bool col_ok = col < vdim;
    const int first = cu[b], last = cu[b + 1];
    float* st = state + ((int64_t) slots[b] * heads + h) * dim * vdim;

    float S[DR];
    const bool resume = pos0[b] > 0;
    #pragma unroll
    for (int i = 0; i < DR; ++i)
    {
        const int r = w + SCAN_WAVES * i;
        S[i] = (resume && col_ok && r < dim) ? st[(int64_t) r * vdim + col] : 0.f;
    }

    for (int n0 = first; n0 < last; n0 += SCAN_TC)
    {
        const int tc = min(SCAN_TC, last - n0);
        __syncthreads();                               // the previous chunk's LDS reads are over
        for (int idx = threadIdx.x; idx < tc * dim; idx += 256)
        {
            const int t = idx / dim, c = idx - t * dim;
            const int64_t n = n0 + t;
            const int hc = h * dim + c;
            qs[idx] = to_f(q[n * q_ld + hc]) * q_scale;
            ks[idx] = to_f(k[n * k_ld + hc]);
            float z = a2_bias ? a2_bias[hc] : 0.f;
            const T* lrow = lr + n * lr_ld;
            const T* arow = a2 + (int64_t) hc * rank;
            for (int r = 0; r < rank; ++r) z += to_f(lrow[r]) * to_f(arow[r]);
            as[idx] = expf(log_sigmoid_f(z) * inv_tau);
        }
        for (int idx = threadIdx.x; idx < tc * 64; idx += 256)
        {
            const int t = idx >> 6, c = vt * 64 + (idx & 63);
            vs[idx] = (c < vdim) ? to_f(v[(int64_t) (n0 + t) * v_ld + h * vdim + c]) : 0.f;
        }
        __syncthreads();
        for (int t = 0; t < tc; ++t)
        {
            const float vv = vs[t * 64 + lane];
            float po = 0.f;
            #pragma unroll
            for (int i = 0; i < DR; ++i)
            {
                const int r = w + SCAN_WAVES * i;
                if (r < dim)
                {
                    S[i] = as[t * dim + r] * S[i] + ks[t * dim + r] * vv;
                    po += qs[t * dim + r] * S[i];
                }
            }
            part[(t * SCAN_WAVES + w) * 64 + lane] = po;
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < tc * 64; idx += 256)
        {
            const int t = idx >> 6, l = idx & 63, c = vt * 64 + l;
            if (c < vdim)
            {
                float s = 0.f;
                #pragma unroll
                for (int ww = 0; ww < SCAN_WAVES; ++ww) s += part[(t * SCAN_WAVES + ww) * 64 + l];
                o[((int64_t) (n0 + t) * heads + h) * vdim + c] = s;
            }
        }
    }
    #pragma unroll
    for (int i = 0; i < DR; ++i)
    {
        const int r = w + SCAN_WAVES * i;
        if (col_ok && r < dim) st[(int64_t) r * vdim + col] = S[i];
    }
}

template <typename T>
__global__ __launch_bounds__(64) void gla_out_kernel(T* __restrict__ out, const float* __restrict__ o, const float* __restrict__ w, const T* __restrict__ g,
                                                     int64_t g_ld, float eps, int heads, int vdim)
{
    const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* orow = o + ((int64_t) n * heads + h) * vdim;
    float ss = 0.f;
    for (int i = lane; i < vdim; i += 64) { float x = orow[i]; ss += x * x; }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float) vdim + eps);
    const T* gr = g + (int64_t) n * g_ld + (int64_t) h * vdim;
    T* dst = out + ((int64_t) n * heads + h) * vdim;
    for (int i = lane; i < vdim; i += 64) dst[i] = from_f<T>(orow[i] * inv * w[i] * silu_f(to_f(gr[i])));
}

extern "C" int exl3_mix_gla_scan(float* o, float* state, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                                 const void* lr, int64_t lr_ld, const void* a2, const float* a2_bias, const int32_t* cu, const int32_t* slots, const int32_t* pos0,
                                 int batch, int heads, int dim, int vdim, int rank, float tau, float q_scale, int dtype, void* stream)
{
    MIX_CHECK(o && state && q && k && v && lr && a2 && cu && slots && pos0, "mix_gla_scan: null pointer");
    MIX_CHECK(batch >= 0 && heads > 0 && dim > 0 && dim <= 256 && vdim > 0 && rank > 0 && tau > 0.f, "mix_gla_scan: sizes out of range (dim %d <= 256)", dim);
    MIX_CHECK(q_ld >= (int64_t) heads * dim && k_ld >= (int64_t) heads * dim && v_ld >= (int64_t) heads * vdim && lr_ld >= rank, "mix_gla_scan: bad row strides");
    if (batch == 0) return EXL3_MIX_OK;
    const dim3 grid(batch, heads, (vdim + 63) / 64);
    const int SCAN_TC = dim > 128 ? 8 : 16;               // tokens staged per chunk: the LDS stays under 64 KB
    const size_t sm = (size_t) (3 * SCAN_TC * dim + SCAN_TC * 64 + SCAN_TC * SCAN_WAVES * 64) * sizeof(float);
    const int dr = (dim + SCAN_WAVES - 1) / SCAN_WAVES;
    #define GLA_SCAN(DRV) hipLaunchKernelGGL((gla_scan_kernel<T, DRV>), grid, dim3(256), sm, (hipStream_t) stream, o, state, (const T*) q, q_ld, (const T*) k, k_ld, \
                                             (const T*) v, v_ld, (const T*) lr, lr_ld, (const T*) a2, a2_bias, cu, slots, pos0, heads, dim, vdim, rank, 1.0f / tau, q_scale, SCAN_TC)
    MIX_DISPATCH_T(dtype,
        if (dr <= 8) GLA_SCAN(8); else if (dr <= 16) GLA_SCAN(16); else if (dr <= 32) GLA_SCAN(32); else GLA_SCAN(64));
    #undef GLA_SCAN
    return mix_check_launch("mix_gla_scan");
}

extern "C" int exl3_mix_gla_out(void* out, const float* o, const float* w, const void* g, int64_t g_ld, float eps, int n, int heads, int vdim, int dtype, void* stream)
{
    MIX_CHECK(out && o && w && g && n >= 0 && heads > 0 && vdim > 0 && g_ld >= (int64_t) heads * vdim, "mix_gla_out: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(gla_out_kernel<T>, dim3(n, heads), dim3(64), 0, (hipStream_t) stream, (T*) out, o, w, (const T*) g, g_ld, eps, heads, vdim));
    return mix_check_launch("mix_gla_out");
}
