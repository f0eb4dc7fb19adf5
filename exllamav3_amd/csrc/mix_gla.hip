// Gated linear attention with a decay per key channel: the token-by-token form (decode, and the exact float32 prefill) and the
// output stage (per-head RMS norm, silu gate).  State, decays, logarithms and every product that enters the recurrence are float32.
//
// Work split of the scan: one workgroup of 4 waves per (sequence, head, block of 64 value columns).  Lane = value column; wave w
// owns the key channels w, w + 4, w + 8, ... (DR of them per lane, in registers).  A chunk of SCAN_TC (16 or 8) tokens is staged in LDS
// (q, k, alpha as float32; alpha computed here from the low-rank decay input), the waves run the recurrence over the chunk without
// a barrier, and the partial outputs of the four waves are added through LDS at the end of the chunk.
#include "mix_common.cuh"

#define SCAN_WAVES 4

// MODE 0: a whole sequence per workgroup, state from / to its slot.
// Long prompts are cut into segments of `seg_len` rows that run in parallel (blockIdx.x = sequence * segs + segment):
// MODE 1: a segment from a zero state, no outputs; leaves its local state and the product of its decays in `seg_state` / `seg_decay`;
// MODE 2: a segment from the state that gla_combine_kernel put into `seg_state`, writes outputs, leaves the slot alone.
#define GLA_WHOLE 0
#define GLA_SEG_LOCAL 1
#define GLA_SEG_FINAL 2

template <typename T, int DR, int MODE>
__global__ __launch_bounds__(256) void gla_scan_kernel(float* __restrict__ o, float* __restrict__ state, const T* __restrict__ q, int64_t q_ld,
                                                       const T* __restrict__ k, int64_t k_ld, const T* __restrict__ v, int64_t v_ld,
                                                       const T* __restrict__ lr, int64_t lr_ld, const T* __restrict__ a2, const float* __restrict__ a2_bias,
                                                       const int32_t* __restrict__ cu, const int32_t* __restrict__ slots, const int32_t* __restrict__ pos0,
                                                       int heads, int dim, int vdim, int rank, float inv_tau, float q_scale, int SCAN_TC,
                                                       int segs, int seg_len, float* __restrict__ seg_state, float* __restrict__ seg_decay)
{
    extern __shared__ float smem[];
    float* qs = smem;                                  // [SCAN_TC][dim]
    float* ks = qs + SCAN_TC * dim;
    float* as = ks + SCAN_TC * dim;
    float* vs = as + SCAN_TC * dim;                    // [SCAN_TC][64]
    float* part = vs + SCAN_TC * 64;                   // [SCAN_TC][SCAN_WAVES][64]
    const int b = (MODE == GLA_WHOLE) ? blockIdx.x : blockIdx.x / segs, h = blockIdx.y, vt = blockIdx.z;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int col = vt * 64 + lane;
    const bool col_ok = col < vdim;
    int first = cu[b], last = cu[b + 1];
    float* st = state + ((int64_t) slots[b] * heads + h) * dim * vdim;
    bool resume = pos0[b] > 0;
    float D[DR];                                       // MODE 1: product of the segment's decays (the same in every lane of a wave)
    if (MODE != GLA_WHOLE)
    {
        const int sg = blockIdx.x - b * segs;
        first += sg * seg_len;
        last = min(last, first + seg_len);
        st = seg_state + ((int64_t) blockIdx.x * heads + h) * dim * vdim;
        resume = (MODE == GLA_SEG_FINAL);
    }

    float S[DR];
    #pragma unroll
    for (int i = 0; i < DR; ++i) D[i] = 1.f;
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
            if (MODE != GLA_SEG_LOCAL) qs[idx] = to_f(q[n * q_ld + hc]) * q_scale;
            ks[idx] = to_f(k[n * k_ld + hc]);
            float z = a2_bias ? a2_bias[hc] : 0.f;
            const T* lrow = lr + n * lr_ld;
            const T* arow = a2 + (int64_t) hc * rank;
            int r = 0;
            for (; r + 8 <= rank; r += 8)                   // eight loads in flight, then the sums (a rolled loop waits for every load in turn)
            {
                float a[8], bb[8];
                #pragma unroll
                for (int e = 0; e < 8; ++e) { a[e] = to_f(lrow[r + e]); bb[e] = to_f(arow[r + e]); }
                #pragma unroll
                for (int e = 0; e < 8; ++e) z += a[e] * bb[e];
            }
            for (; r < rank; ++r) z += to_f(lrow[r]) * to_f(arow[r]);
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
                    const float a = as[t * dim + r];
                    S[i] = a * S[i] + ks[t * dim + r] * vv;
                    if (MODE == GLA_SEG_LOCAL) D[i] *= a; else po += qs[t * dim + r] * S[i];
                }
            }
            if (MODE != GLA_SEG_LOCAL) part[(t * SCAN_WAVES + w) * 64 + lane] = po;
        }
        if (MODE == GLA_SEG_LOCAL) continue;
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
    if (MODE == GLA_SEG_FINAL) return;
    #pragma unroll
    for (int i = 0; i < DR; ++i)
    {
        const int r = w + SCAN_WAVES * i;
        if (col_ok && r < dim) st[(int64_t) r * vdim + col] = S[i];
        if (MODE == GLA_SEG_LOCAL && vt == 0 && lane == 0 && r < dim) seg_decay[((int64_t) blockIdx.x * heads + h) * dim + r] = D[i];
    }
}

// Between the two segment passes: walks a sequence's segments in order.  seg_state[s] (the segment's local state) is replaced by the state the
// segment starts from, S_start[s+1] = diag(decay[s]) S_start[s] + local[s]; the state after the last segment goes to the sequence's slot.
__global__ __launch_bounds__(256) void gla_combine_kernel(float* __restrict__ state, float* __restrict__ seg_state, const float* __restrict__ seg_decay,
                                                          const int32_t* __restrict__ cu, const int32_t* __restrict__ slots, const int32_t* __restrict__ pos0,
                                                          int heads, int dim, int vdim, int segs, int seg_len)
{
    const int b = blockIdx.x, h = blockIdx.y;
    const int64_t per = (int64_t) dim * vdim;
    const int used = min(segs, (cu[b + 1] - cu[b] + seg_len - 1) / seg_len);
    float* st = state + ((int64_t) slots[b] * heads + h) * per;
    const bool resume = pos0[b] > 0;
    for (int64_t e = (int64_t) blockIdx.z * 256 + threadIdx.x; e < per; e += (int64_t) gridDim.z * 256)
    {
        const int r = (int) (e / vdim);
        float S = resume ? st[e] : 0.f;
        for (int sg = 0; sg < used; ++sg)
        {
            const int64_t blk = ((int64_t) b * segs + sg) * heads + h;
            const float local = seg_state[blk * per + e];
            seg_state[blk * per + e] = S;
            S = seg_decay[blk * dim + r] * S + local;
        }
        st[e] = S;
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

template <int MODEV>
static int gla_launch(float* o, float* state, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                      const void* lr, int64_t lr_ld, const void* a2, const float* a2_bias, const int32_t* cu, const int32_t* slots, const int32_t* pos0,
                      int batch, int heads, int dim, int vdim, int rank, float tau, float q_scale, int dtype, void* stream,
                      int segs, int seg_len, float* seg_state, float* seg_decay)
{
    MIX_CHECK(o && state && q && k && v && lr && a2 && cu && slots && pos0, "mix_gla_scan: null pointer");
    MIX_CHECK(batch >= 0 && heads > 0 && dim > 0 && dim <= 256 && vdim > 0 && rank > 0 && tau > 0.f, "mix_gla_scan: sizes out of range (dim %d <= 256)", dim);
    MIX_CHECK(q_ld >= (int64_t) heads * dim && k_ld >= (int64_t) heads * dim && v_ld >= (int64_t) heads * vdim && lr_ld >= rank, "mix_gla_scan: bad row strides");
    if (batch == 0) return EXL3_MIX_OK;
    const dim3 grid(batch * segs, heads, (vdim + 63) / 64);
    const int SCAN_TC = dim > 128 ? 8 : 16;               // tokens staged per chunk: the LDS stays under 64 KB
    const size_t sm = (size_t) (3 * SCAN_TC * dim + SCAN_TC * 64 + SCAN_TC * SCAN_WAVES * 64) * sizeof(float);
    const int dr = (dim + SCAN_WAVES - 1) / SCAN_WAVES;
    #define GLA_SCAN(DRV) hipLaunchKernelGGL((gla_scan_kernel<T, DRV, MODEV>), grid, dim3(256), sm, (hipStream_t) stream, o, state, (const T*) q, q_ld, (const T*) k, k_ld, \
                                             (const T*) v, v_ld, (const T*) lr, lr_ld, (const T*) a2, a2_bias, cu, slots, pos0, heads, dim, vdim, rank, 1.0f / tau, q_scale, SCAN_TC, \
                                             segs, seg_len, seg_state, seg_decay)
    MIX_DISPATCH_T(dtype,
        if (dr <= 8) GLA_SCAN(8); else if (dr <= 16) GLA_SCAN(16); else if (dr <= 32) GLA_SCAN(32); else GLA_SCAN(64));
    #undef GLA_SCAN
    return mix_check_launch("mix_gla_scan");
}

extern "C" int exl3_mix_gla_scan(float* o, float* state, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                                 const void* lr, int64_t lr_ld, const void* a2, const float* a2_bias, const int32_t* cu, const int32_t* slots, const int32_t* pos0,
                                 int batch, int heads, int dim, int vdim, int rank, float tau, float q_scale, int dtype, void* stream)
{
    return gla_launch<GLA_WHOLE>(o, state, q, q_ld, k, k_ld, v, v_ld, lr, lr_ld, a2, a2_bias, cu, slots, pos0, batch, heads, dim, vdim, rank, tau, q_scale, dtype, stream,
                                 1, 0, nullptr, nullptr);
}

extern "C" int exl3_mix_gla_segmented(float* o, float* state, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                                      const void* lr, int64_t lr_ld, const void* a2, const float* a2_bias, const int32_t* cu, const int32_t* slots, const int32_t* pos0,
                                      int batch, int heads, int dim, int vdim, int rank, float tau, float q_scale, int segs, int seg_len,
                                      float* seg_state, float* seg_decay, int dtype, void* stream)
{
    MIX_CHECK(segs >= 1 && seg_len >= 1 && seg_state && seg_decay, "mix_gla_segmented: bad segment arguments");
    int rc = gla_launch<GLA_SEG_LOCAL>(o, state, q, q_ld, k, k_ld, v, v_ld, lr, lr_ld, a2, a2_bias, cu, slots, pos0, batch, heads, dim, vdim, rank, tau, q_scale, dtype,
                                       stream, segs, seg_len, seg_state, seg_decay);
    if (rc || batch == 0) return rc;
    const int64_t per = (int64_t) dim * vdim;
    hipLaunchKernelGGL(gla_combine_kernel, dim3(batch, heads, (unsigned) ((per + 1023) / 1024)), dim3(256), 0, (hipStream_t) stream, state, seg_state, seg_decay, cu, slots, pos0,
                       heads, dim, vdim, segs, seg_len);
    if ((rc = mix_check_launch("mix_gla_segmented (combine)"))) return rc;
    return gla_launch<GLA_SEG_FINAL>(o, state, q, q_ld, k, k_ld, v, v_ld, lr, lr_ld, a2, a2_bias, cu, slots, pos0, batch, heads, dim, vdim, rank, tau, q_scale, dtype,
                                     stream, segs, seg_len, seg_state, seg_decay);
}

extern "C" int exl3_mix_gla_out(void* out, const float* o, const float* w, const void* g, int64_t g_ld, float eps, int n, int heads, int vdim, int dtype, void* stream)
{
    MIX_CHECK(out && o && w && g && n >= 0 && heads > 0 && vdim > 0 && g_ld >= (int64_t) heads * vdim, "mix_gla_out: bad arguments");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(gla_out_kernel<T>, dim3(n, heads), dim3(64), 0, (hipStream_t) stream, (T*) out, o, w, (const T*) g, g_ld, eps, heads, vdim));
    return mix_check_launch("mix_gla_out");
}
