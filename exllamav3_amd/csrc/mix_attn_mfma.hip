// Prefill of the sliding-window sink attention on the matrix cores (bfloat16 activations): scores = Q K^T and the weighted sum P V with
// v_mfma_f32_16x16x32_bf16, scores, running maximum, exponentials and sums in float32; the softmax starts from the sink, so the sink is one
// more term of the denominator and nothing else.
//
// One workgroup = 128 query rows of one sequence and one head, 8 waves of 16 rows.  Key tiles of KT = 64 rows (32 for the largest heads, where
// 64 would not fit 64 KB of LDS) are staged in LDS once for the eight waves: K as stored, V transposed (so that both are read as 16-byte contraction groups).  MFMA operand lane (g = lane / 16, c = lane % 16)
// holds row / column c and contraction slots 8g .. 8g+7; result lane (g, c) holds rows 4g .. 4g+3 of column c.  A wave's P tile goes
// through its own LDS patch from the result layout to the operand layout.  Only the key tiles that intersect the window of the block's
// rows are visited, and a wave skips the tiles outside its own rows' windows.
#include "mix_common.cuh"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define AM_ROWS 128
#define AM_THREADS 512
#define AM_PAD 8

// KD: contraction steps of 32 over the (zero-padded) head dim; NV: 16-column tiles of the (padded) value dim.
template <int KD, int NV, int AM_KEYS>
__global__ __launch_bounds__(AM_THREADS) void attn_prefill_mfma_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ q, int64_t q_ld, const bf16_t* __restrict__ k,
                                                                int64_t k_ld, const bf16_t* __restrict__ v_norm, const bf16_t* __restrict__ gate, int64_t gate_ld,
                                                                const float* __restrict__ sink, const int32_t* __restrict__ cu,
                                                                int heads, int kv_heads, int dim, int vdim, float scale, int window, int k_vec, int v_vec)
{
    constexpr int DP = KD * 32, KS = DP + AM_PAD, VS = AM_KEYS + AM_PAD, PS = AM_KEYS + AM_PAD;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    uint16_t* k_lds = (uint16_t*) smem_raw;                       // [AM_KEYS][KS]
    uint16_t* vt_lds = k_lds + AM_KEYS * KS;                      // [NV * 16][VS]   (value column, key)
    uint16_t* p_lds = vt_lds + NV * 16 * VS;                      // [8 waves][16][PS]

    const int b = blockIdx.y, h = blockIdx.z;
    const int first = cu[b], len = cu[b + 1] - first;
    const int q0 = blockIdx.x * AM_ROWS;
    if (q0 >= len) return;
    const int kvh = h / (heads / kv_heads);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, g = lane >> 4, c = lane & 15;
    uint16_t* pw = p_lds + w * 16 * PS;

    // this wave's 16 query rows as A operands (rows beyond the sequence read row len-1: computed and never stored)
    const int qrow_a = min(q0 + w * 16 + c, len - 1);
    bf16x8 qf[KD];
    #pragma unroll
    for (int s = 0; s < KD; ++s)
    {
        union { bf16x8 v; uint16_t u[8]; } t;
        #pragma unroll
        for (int e = 0; e < 8; ++e)
        {
            const int col = s * 32 + g * 8 + e;
            t.u[e] = col < dim ? q[(int64_t) (first + qrow_a) * q_ld + (int64_t) h * dim + col].u : (uint16_t) 0;
        }
        qf[s] = t.v;
    }
    const int wq_lo = q0 + w * 16, wq_hi = min(q0 + w * 16 + 15, len - 1);           // this wave's rows
    const bool wave_live = wq_lo < len;

    const float sk = sink ? sink[h] : -1e30f;
    float m[4], l[4];
    f32x4 acc[NV];
    #pragma unroll
    for (int i = 0; i < 4; ++i) { m[i] = sk; l[i] = sink ? 1.0f : 0.0f; }
    #pragma unroll
    for (int t = 0; t < NV; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int blk_hi = min(q0 + AM_ROWS - 1, len - 1);
    const int j_begin = (max(0, q0 - window + 1) / AM_KEYS) * AM_KEYS;
    for (int j0 = j_begin; j0 <= blk_hi; j0 += AM_KEYS)
    {
        __syncthreads();                                           // the previous tile's operand reads are over
        // stage K [32][DP] (zero beyond dim / len) and V^T [vdim][32]
        for (int idx = threadIdx.x; idx < AM_KEYS * (DP / 8); idx += AM_THREADS)
        {
            const int r = idx / (DP / 8), cg = idx - r * (DP / 8);
            const int j = j0 + r;
            const bf16_t* src = k + (int64_t) (first + min(j, len - 1)) * k_ld + (int64_t) kvh * dim + cg * 8;
            union { uint4 v; uint16_t u[8]; } t;
            if (k_vec && j < len && cg * 8 + 8 <= dim) t.v = *(const uint4*) src;          // 16-byte rows (host-checked alignment)
            else
            {
                #pragma unroll
                for (int e = 0; e < 8; ++e) t.u[e] = (j < len && cg * 8 + e < dim) ? src[e].u : (uint16_t) 0;
            }
            *(uint4*) (k_lds + r * KS + cg * 8) = t.v;
        }
        for (int idx = threadIdx.x; idx < AM_KEYS * NV * 2; idx += AM_THREADS)
        {
            const int cg = idx / AM_KEYS, r = idx - cg * AM_KEYS;               // consecutive lanes: consecutive keys of one column group (LDS stores side by side)
            const int j = j0 + r;
            const bf16_t* src = v_norm + ((int64_t) (first + min(j, len - 1)) * kv_heads + kvh) * vdim + cg * 8;
            union { uint4 v; uint16_t u[8]; } t;
            if (v_vec && j < len && cg * 8 + 8 <= vdim) t.v = *(const uint4*) src;
            else
            {
                #pragma unroll
                for (int e = 0; e < 8; ++e) t.u[e] = (j < len && cg * 8 + e < vdim) ? src[e].u : (uint16_t) 0;
            }
            #pragma unroll
            for (int e = 0; e < 8; ++e) vt_lds[(cg * 8 + e) * VS + r] = t.u[e];
        }
        __syncthreads();
        // tiles wholly outside this wave's windows: nothing to add (uniform per wave; the barriers above are still met)
        const bool skip = !wave_live || j0 > wq_hi || j0 + AM_KEYS - 1 < wq_lo - window + 1;
        if (!skip)
        {
            constexpr int NS = AM_KEYS / 16;                                   // 16-key score tiles
            f32x4 sc[NS];
            #pragma unroll
            for (int u = 0; u < NS; ++u) sc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
            #pragma unroll
            for (int s = 0; s < KD; ++s)
            {
                #pragma unroll
                for (int u = 0; u < NS; ++u)
                {
                    const bf16x8 kf = *(const bf16x8*) (k_lds + (u * 16 + c) * KS + s * 32 + g * 8);
                    sc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[s], kf, sc[u], 0, 0, 0);
                }
            }
            float corr[4];
            #pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                const int qi = q0 + w * 16 + g * 4 + i;                       // this result row's position
                float sv[NS];
                float mx = -INFINITY;
                #pragma unroll
                for (int u = 0; u < NS; ++u)
                {
                    const int j = j0 + u * 16 + c;
                    const bool ok = j <= qi && qi - j < window && qi < len;
                    sv[u] = ok ? sc[u][i] * scale : -INFINITY;
                    mx = fmaxf(mx, sv[u]);
                }
                #pragma unroll
                for (int o = 8; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
                const float mn = fmaxf(m[i], mx);                              // finite: m starts at the sink or at -1e30
                float sum = 0.f;
                #pragma unroll
                for (int u = 0; u < NS; ++u)
                {
                    const float pv = expf(sv[u] - mn);                         // masked: exp(-inf) = 0
                    sum += pv;
                    pw[(g * 4 + i) * PS + u * 16 + c] = from_f<bf16_t>(pv).u;
                }
                #pragma unroll
                for (int o = 8; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
                corr[i] = expf(m[i] - mn);
                l[i] = l[i] * corr[i] + sum;
                m[i] = mn;
            }
            #pragma unroll
            for (int t = 0; t < NV; ++t)
            {
                #pragma unroll
                for (int i = 0; i < 4; ++i) acc[t][i] *= corr[i];
            }
            __builtin_amdgcn_wave_barrier();                                   // LDS serves a wave's accesses in order: its own P stores are visible to the reads below
            #pragma unroll
            for (int kk = 0; kk < AM_KEYS / 32; ++kk)
            {
                const bf16x8 pa8 = *(const bf16x8*) (pw + c * PS + kk * 32 + g * 8);
                #pragma unroll
                for (int t = 0; t < NV; ++t)
                {
                    const bf16x8 vb = *(const bf16x8*) (vt_lds + (t * 16 + c) * VS + kk * 32 + g * 8);
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa8, vb, acc[t], 0, 0, 0);
                }
            }
        }
    }
    if (!wave_live) return;
    #pragma unroll
    for (int i = 0; i < 4; ++i)
    {
        const int qi = q0 + w * 16 + g * 4 + i;
        if (qi >= len) continue;
        const int64_t n = first + qi;
        const float gt = gate ? sigmoid_f(to_f(gate[n * gate_ld + h])) : 1.0f;
        const float f = (l[i] > 0.f ? 1.0f / l[i] : 0.f) * gt;
        #pragma unroll
        for (int t = 0; t < NV; ++t)
        {
            const int col = t * 16 + c;
            if (col < vdim) out[(n * heads + h) * vdim + col] = from_f<bf16_t>(acc[t][i] * f);
        }
    }
}

extern "C" int exl3_mix_attn_prefill_mfma(void* out, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v_norm,
                                          const void* gate, int64_t gate_ld, const float* sink, const int32_t* cu,
                                          int batch, int max_rows, int heads, int kv_heads, int dim, int vdim, float scale, int window, void* stream)
{
    MIX_CHECK(out && q && k && v_norm && cu, "mix_attn_prefill_mfma: null pointer");
    MIX_CHECK(batch >= 0 && max_rows >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && heads <= 65535 && batch <= 65535,
              "mix_attn_prefill_mfma: heads %d / kv_heads %d / batch %d", heads, kv_heads, batch);
    MIX_CHECK(dim > 0 && dim <= 256 && vdim > 0 && vdim <= 256 && window > 0, "mix_attn_prefill_mfma: dim %d and vdim %d must be <= 256", dim, vdim);
    MIX_CHECK(q_ld >= (int64_t) heads * dim && k_ld >= (int64_t) kv_heads * dim && (!gate || gate_ld >= heads), "mix_attn_prefill_mfma: bad row strides");
    if (batch == 0 || max_rows == 0) return EXL3_MIX_OK;
    const dim3 grid((max_rows + AM_ROWS - 1) / AM_ROWS, batch, heads);
    const int k_vec = ((uintptr_t) k % 16 == 0) && (k_ld % 8 == 0) && (dim % 8 == 0);
    const int v_vec = ((uintptr_t) v_norm % 16 == 0) && (vdim % 8 == 0);
    #define AM_LDS(KDV, NVV, KTV) ((size_t) (KTV * (KDV * 32 + AM_PAD) + NVV * 16 * (KTV + AM_PAD) + (AM_THREADS / 64) * 16 * (KTV + AM_PAD)) * sizeof(uint16_t))
    #define AM_LAUNCH(KDV, NVV, KTV) do { \
        static_assert(AM_LDS(KDV, NVV, KTV) <= 65536, "tile does not fit the LDS"); \
        hipLaunchKernelGGL((attn_prefill_mfma_kernel<KDV, NVV, KTV>), grid, dim3(AM_THREADS), AM_LDS(KDV, NVV, KTV), (hipStream_t) stream, (bf16_t*) out, (const bf16_t*) q, q_ld, \
                           (const bf16_t*) k, k_ld, (const bf16_t*) v_norm, (const bf16_t*) gate, gate_ld, sink, cu, heads, kv_heads, dim, vdim, scale, window, k_vec, v_vec); } while (0)
    const int kd = (dim + 31) / 32, nv = (vdim + 15) / 16;
    if (kd <= 2)      { if (nv <= 4) AM_LAUNCH(2, 4, 64); else if (nv <= 8) AM_LAUNCH(2, 8, 64); else AM_LAUNCH(2, 16, 64); }
    else if (kd <= 4) { if (nv <= 4) AM_LAUNCH(4, 4, 64); else if (nv <= 8) AM_LAUNCH(4, 8, 64); else AM_LAUNCH(4, 16, 32); }
    else              { if (nv <= 4) AM_LAUNCH(8, 4, 64); else if (nv <= 8) AM_LAUNCH(8, 8, 32); else AM_LAUNCH(8, 16, 32); }
    #undef AM_LDS
    #undef AM_LAUNCH
    return mix_check_launch("mix_attn_prefill_mfma");
}
