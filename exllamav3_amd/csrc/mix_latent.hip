// Latent attention: keys and values of all heads are up-projections of one low-rank latent c per token, plus one rotated key part shared by
// the heads, and only [c | k_rot] is cached (a ring of `window` entries per slot).
//
//   latent_prep     RMS norm of the latent (float32), rotary positions (angles, cos and sin in float32; interleaved pairs; per-pair
//                   frequencies and one magnitude given by the caller, so any frequency scaling is the caller's table) on the shared key part
//                   and on the rotated part of every query head, the step's [c | k_rot] rows and the ring entries of the rows the window keeps
//   latent_fill_k   prompt steps: the shared rotated part copied behind every head's up-projected key
//   latent_decode   decode steps in the ABSORBED form: the query is carried into the latent space (q_lat = W_uk^T q per head, a vendor product), the
//                   cached [c | k_rot] rows are the keys of every head and c is also the value; the result is a weighted latent per head that the
//                   caller up-projects with W_uv.  Scores, softmax and sums are the float32 row worker of mix_attn_row.cuh.
//   latent_decode_mfma   the same on the matrix cores (bfloat16): all heads of a sequence score the SAME cached rows, so sixteen heads are the
//                   sixteen columns of one MFMA tile and every cached row is read once per sixteen heads instead of once per head.  The keys of a
//                   sequence are split over workgroups whose four waves share the rows' columns; a second kernel merges the partial sums (and adds the sink).
#include "mix_common.cuh"
#include "mix_attn_row.cuh"

template <typename T>
__global__ __launch_bounds__(256) void latent_prep_kernel(T* __restrict__ ckr, T* __restrict__ ring, const T* __restrict__ dkv, int64_t dkv_ld,
                                                          const float* __restrict__ norm_w, T* __restrict__ q, int64_t q_ld,
                                                          const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                                                          const int32_t* __restrict__ slots, const int32_t* __restrict__ len_after,
                                                          const float* __restrict__ freq, float mag, float eps,
                                                          int heads, int dim, int rot_dim, int rot_dims, int rank, int window)
{
    __shared__ float red[4];
    extern __shared__ float trig[];                            // [pairs][2]: cos, sin of the row's position, computed once for the key part and every head
    const int n = blockIdx.x;
    const int b = tok_seq[n], pos = tok_pos[n];
    const bool keep = pos >= len_after[b] - window;
    const int row = rank + rot_dim;
    const T* src = dkv + (int64_t) n * dkv_ld;
    T* dst = ckr + (int64_t) n * row;
    T* rg = ring + ((int64_t) slots[b] * window + (pos % window)) * row;
    float ss = 0.f;
    for (int i = threadIdx.x; i < rank; i += 256) { const float v = to_f(src[i]); ss += v * v; }
    ss = block_sum<4>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float) rank + eps);
    for (int i = threadIdx.x; i < rank; i += 256)
    {
        const T o = from_f<T>(to_f(src[i]) * inv * norm_w[i]);
        dst[i] = o;
        if (keep) rg[i] = o;
    }
    const int pairs = rot_dims / 2;
    const float p = (float) pos;
    for (int i = threadIdx.x; i < pairs; i += 256)
    {
        float sn, cs;
        sincosf(p * freq[i], &sn, &cs);
        trig[2 * i] = cs * mag; trig[2 * i + 1] = sn * mag;
    }
    __syncthreads();
    // the shared key part: rotated pairs, then what lies beyond rot_dims unchanged
    for (int i = threadIdx.x; i < pairs; i += 256)
    {
        const float cs = trig[2 * i], sn = trig[2 * i + 1];
        const float u = to_f(src[rank + 2 * i]), v = to_f(src[rank + 2 * i + 1]);
        const T o0 = from_f<T>(u * cs - v * sn), o1 = from_f<T>(v * cs + u * sn);
        dst[rank + 2 * i] = o0; dst[rank + 2 * i + 1] = o1;
        if (keep) { rg[rank + 2 * i] = o0; rg[rank + 2 * i + 1] = o1; }
    }
    for (int i = rot_dims + threadIdx.x; i < rot_dim; i += 256)
    {
        const T o = src[rank + i];
        dst[rank + i] = o;
        if (keep) rg[rank + i] = o;
    }
    // the rotated part of every query head, in place
    T* qr = q + (int64_t) n * q_ld;
    for (int t = threadIdx.x; t < heads * pairs; t += 256)
    {
        const int h = t / pairs, i = t - h * pairs;
        const float cs = trig[2 * i], sn = trig[2 * i + 1];
        T* e = qr + (int64_t) h * (dim + rot_dim) + dim + 2 * i;
        const float u = to_f(e[0]), v = to_f(e[1]);
        e[0] = from_f<T>(u * cs - v * sn);
        e[1] = from_f<T>(v * cs + u * sn);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void latent_fill_k_kernel(T* __restrict__ k, int64_t k_ld, const T* __restrict__ ckr, int heads, int dim, int rot_dim, int rank)
{
    const int n = blockIdx.x;
    const T* src = ckr + (int64_t) n * (rank + rot_dim) + rank;
    T* kr = k + (int64_t) n * k_ld;
    for (int t = threadIdx.x; t < heads * rot_dim; t += 256)
    {
        const int h = t / rot_dim, i = t - h * rot_dim;
        kr[(int64_t) h * (dim + rot_dim) + dim + i] = src[i];
    }
}

template <typename T, int MAXV>
__global__ __launch_bounds__(64 * AT_WAVES) void latent_decode_kernel(T* __restrict__ o_lat, int64_t o_row, int64_t o_head, const T* __restrict__ q_lat, int64_t ql_row,
                                                                      int64_t ql_head, const T* __restrict__ q, int64_t q_ld, const T* __restrict__ ring,
                                                                      const float* __restrict__ sink, const int32_t* __restrict__ slots,
                                                                      const int32_t* __restrict__ len_after, int dim, int rot_dim, int rank, float scale, int window)
{
    extern __shared__ float smem[];
    const int n = blockIdx.x, h = blockIdx.y;
    const int count = min(len_after[n], window);
    const int row = rank + rot_dim;
    const T* kb = ring + (int64_t) slots[n] * window * row;
    attn_row<T, MAXV>(o_lat + (int64_t) n * o_row + (int64_t) h * o_head, q_lat + (int64_t) n * ql_row + (int64_t) h * ql_head,
                      q + (int64_t) n * q_ld + (int64_t) h * (dim + rot_dim) + dim, rank, kb, row, kb, row, count, row, rank, scale,
                      sink != nullptr, sink ? sink[h] : 0.f, 1.0f, rows_are_16_byte(kb, (int64_t) row, row), smem);
}

extern "C" int exl3_mix_latent_prep(void* ckr, void* ring, const void* dkv, int64_t dkv_ld, const float* norm_w, void* q, int64_t q_ld,
                                    const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* slots, const int32_t* len_after,
                                    const float* freq, float mag, float eps, int n, int heads, int dim, int rot_dim, int rot_dims, int rank, int window,
                                    int dtype, void* stream)
{
    MIX_CHECK(ckr && ring && dkv && norm_w && q && tok_seq && tok_pos && slots && len_after && freq, "mix_latent_prep: null pointer");
    MIX_CHECK(n >= 0 && heads > 0 && dim >= 0 && rot_dim >= 0 && rank > 0 && window > 0, "mix_latent_prep: bad sizes");
    MIX_CHECK(rot_dims >= 0 && rot_dims <= rot_dim && rot_dims % 2 == 0, "mix_latent_prep: %d rotated dimensions of %d", rot_dims, rot_dim);
    MIX_CHECK(dkv_ld >= rank + rot_dim && q_ld >= (int64_t) heads * (dim + rot_dim), "mix_latent_prep: bad row strides");
    if (n == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(latent_prep_kernel<T>, dim3(n), dim3(256), (size_t) (rot_dims + 2) * sizeof(float), (hipStream_t) stream, (T*) ckr, (T*) ring, (const T*) dkv, dkv_ld, norm_w,
                                             (T*) q, q_ld, tok_seq, tok_pos, slots, len_after, freq, mag, eps, heads, dim, rot_dim, rot_dims, rank, window));
    return mix_check_launch("mix_latent_prep");
}

extern "C" int exl3_mix_latent_fill_k(void* k, int64_t k_ld, const void* ckr, int n, int heads, int dim, int rot_dim, int rank, int dtype, void* stream)
{
    MIX_CHECK(k && ckr && n >= 0 && heads > 0 && dim >= 0 && rot_dim >= 0 && rank > 0 && k_ld >= (int64_t) heads * (dim + rot_dim), "mix_latent_fill_k: bad arguments");
    if (n == 0 || rot_dim == 0) return EXL3_MIX_OK;
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(latent_fill_k_kernel<T>, dim3(n), dim3(256), 0, (hipStream_t) stream, (T*) k, k_ld, (const T*) ckr, heads, dim, rot_dim, rank));
    return mix_check_launch("mix_latent_fill_k");
}

extern "C" int exl3_mix_latent_decode(void* o_lat, int64_t o_row, int64_t o_head, const void* q_lat, int64_t ql_row, int64_t ql_head, const void* q, int64_t q_ld,
                                      const void* ring, const float* sink, const int32_t* slots, const int32_t* len_after,
                                      int n, int heads, int dim, int rot_dim, int rank, float scale, int window, int dtype, void* stream)
{
    MIX_CHECK(o_lat && q_lat && q && ring && slots && len_after, "mix_latent_decode: null pointer");
    MIX_CHECK(n >= 0 && heads > 0 && heads <= 65535 && dim >= 0 && rot_dim >= 0 && rank > 0 && rank <= 1024 && rank + rot_dim <= 4096 && window > 0,
              "mix_latent_decode: rank %d (<= 1024) / rot_dim %d / window %d out of range", rank, rot_dim, window);
    MIX_CHECK(q_ld >= (int64_t) heads * (dim + rot_dim), "mix_latent_decode: bad row stride");
    if (n == 0) return EXL3_MIX_OK;
    const int mv = (rank + 63) / 64;
    const int mvt = mv == 1 ? 1 : (mv == 2 ? 2 : (mv <= 4 ? 4 : (mv <= 8 ? 8 : 16)));
    const size_t sm = (size_t) (rank + rot_dim + AT_WAVES * 64 + AT_WAVES * (2 + mvt * 64)) * sizeof(float);
    #define LD_LAUNCH(MV) hipLaunchKernelGGL((latent_decode_kernel<T, MV>), dim3(n, heads), dim3(64 * AT_WAVES), sm, (hipStream_t) stream, (T*) o_lat, o_row, o_head, \
                                             (const T*) q_lat, ql_row, ql_head, (const T*) q, q_ld, (const T*) ring, sink, slots, len_after, dim, rot_dim, rank, scale, window)
    MIX_DISPATCH_T(dtype,
        if (mv == 1) LD_LAUNCH(1); else if (mv == 2) LD_LAUNCH(2); else if (mv <= 4) LD_LAUNCH(4); else if (mv <= 8) LD_LAUNCH(8); else LD_LAUNCH(16));
    #undef LD_LAUNCH
    return mix_check_launch("mix_latent_decode");
}

// ---- decode on the matrix cores ---------------------------------------------------------------------------------------------------------------
// One workgroup of four waves = one split of one sequence's cached rows x one group of 16 heads.  v_mfma_f32_16x16x32_bf16 operand lane (g = lane / 16,
// c = lane % 16) holds row / column c and contraction slots 8g .. 8g+7; result lane (g, c) holds rows 4g .. 4g+3 of column c.
//   scores, transposed: S^T = K Q^T.  A = 16 cached rows (lane: row c, 16 bytes straight from the ring, no staging), B = the 16 heads' absorbed queries
//   [q_lat | q_rot] (registers, loaded once).  A lane then holds the scores of ONE head, so the running maximum and sum are per-lane scalars.
//   O^T = C^T P^T over tiles of 32 keys: the score registers of two 16-key tiles are the B operand as they stand when contraction slot (g, e) means key
//   4g + e of the first tile (e < 4) or of the second (e >= 4); A = the latent columns of the same rows, transposed through LDS (the rows are in registers
//   already: they were the A operands of the scores).
// The four waves split the COLUMNS of the cached rows: wave w loads a quarter of every row (and one of the up to two 32-column steps behind the padded
// latent), contributes that quarter's share of the scores -- summed through LDS in a fixed order, so every wave holds the same scores and repeats the few
// softmax steps -- and owns the same quarter of the latent columns in the second product: a quarter of the accumulators, its own rows of C^T in LDS.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
#define LM_KEYS 32
#define LM_VS (LM_KEYS + 8)
#define LM_WAVES 4

template <int NV>
__global__ __launch_bounds__(64 * LM_WAVES) void latent_decode_mfma_kernel(float* __restrict__ part_o, float* __restrict__ part_ml, const bf16_t* __restrict__ q_lat,
                                                                           int64_t ql_row, int64_t ql_head, const bf16_t* __restrict__ q, int64_t q_ld,
                                                                           const bf16_t* __restrict__ ring, const int32_t* __restrict__ slots,
                                                                           const int32_t* __restrict__ len_after, int heads, int dim, int rot_dim, int rank, float scale,
                                                                           int window, int keys_per_split, int q_vec)
{
    constexpr int KDW = NV / 8;                                 // 32-column steps of the padded latent per wave
    constexpr int NVW = NV / 4;                                 // 16-column tiles of the latent per wave
    constexpr int NS = KDW + 1;                                 // + one step behind the padded latent (columns NV * 16 + 32 w ..), empty for most waves
    __shared__ __attribute__((aligned(16))) uint16_t vt[NV * 16 * LM_VS];        // [latent column][key of the tile]; wave w owns rows w * NV * 4 ..
    __shared__ __attribute__((aligned(16))) float sp[LM_WAVES][2][64][4];         // the waves' shares of the scores
    const int sp_i = blockIdx.x, hg = blockIdx.y, n = blockIdx.z, splits = gridDim.x;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, g = lane >> 4, c = lane & 15;
    const int count = min(len_after[n], window);
    const int k_begin = sp_i * keys_per_split, k_end = min(count, k_begin + keys_per_split);
    const int row = rank + rot_dim;
    const bf16_t* kb = ring + (int64_t) slots[n] * window * row;
    const int head = hg * 16 + c;
    const bool head_ok = head < heads;
    const int64_t pidx = ((int64_t) n * splits + sp_i) * heads + head;
    if (k_begin >= k_end)
    {
        if (w == 0 && head_ok && g == 0) { part_ml[pidx * 2] = -INFINITY; part_ml[pidx * 2 + 1] = 0.f; }
        return;
    }
    // this wave's steps: first column of step i (rank and row are multiples of 8: a group of 8 columns lies in one part of the row or beyond it)
    int col_of[NS];
    #pragma unroll
    for (int i = 0; i < NS; ++i) col_of[i] = (i < KDW ? (w * KDW + i) * 32 : NV * 16 + w * 32) + g * 8;
    bf16x8 qf[NS];
    #pragma unroll
    for (int i = 0; i < NS; ++i)
    {
        union { bf16x8 v; uint4 x; uint16_t u[8]; } t;
        const int c0 = col_of[i];
        const bf16_t* src = c0 < rank ? q_lat + (int64_t) n * ql_row + (int64_t) head * ql_head + c0
                                      : q + (int64_t) n * q_ld + (int64_t) head * (dim + rot_dim) + dim + (c0 - rank);
        if (!head_ok || c0 >= row) t.x = uint4{0u, 0u, 0u, 0u};
        else if (q_vec) t.x = *(const uint4*) src;                // 16-byte groups (host-checked alignment)
        else
        {
            #pragma unroll
            for (int e = 0; e < 8; ++e) t.u[e] = src[e].u;
        }
        qf[i] = t.v;
    }
    float m = -1e30f, l = 0.f;
    f32x4 acc[NVW];
    #pragma unroll
    for (int t = 0; t < NVW; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int j0 = k_begin; j0 < k_end; j0 += LM_KEYS)
    {
        union kreg { bf16x8 v; uint4 x; uint16_t e[8]; };
        kreg kf[2][NS];
        #pragma unroll
        for (int u = 0; u < 2; ++u)
        {
            const int jr = min(j0 + u * 16 + c, count - 1);       // rows past the split are read (they exist) and masked below
            const bf16_t* kr = kb + (int64_t) jr * row;
            #pragma unroll
            for (int i = 0; i < NS; ++i) kf[u][i].x = col_of[i] < row ? *(const uint4*) (kr + col_of[i]) : uint4{0u, 0u, 0u, 0u};
        }
        __syncthreads();                                           // the previous tile's reads of sp and vt are over
        #pragma unroll
        for (int u = 0; u < 2; ++u)
        {
            f32x4 part = f32x4{0.f, 0.f, 0.f, 0.f};
            #pragma unroll
            for (int i = 0; i < NS; ++i) part = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[u][i].v, qf[i], part, 0, 0, 0);
            *(f32x4*) sp[w][u][lane] = part;
            #pragma unroll
            for (int i = 0; i < KDW; ++i)
            {
                #pragma unroll
                for (int e = 0; e < 8; ++e) vt[(col_of[i] + e) * LM_VS + u * 16 + c] = kf[u][i].e[e];
            }
        }
        __syncthreads();
        f32x4 sc[2];
        #pragma unroll
        for (int u = 0; u < 2; ++u)
            sc[u] = (*(const f32x4*) sp[0][u][lane] + *(const f32x4*) sp[1][u][lane]) + (*(const f32x4*) sp[2][u][lane] + *(const f32x4*) sp[3][u][lane]);
        float mx = -INFINITY;
        #pragma unroll
        for (int u = 0; u < 2; ++u)
        {
            #pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                const bool ok = j0 + u * 16 + g * 4 + i < k_end;
                sc[u][i] = ok ? sc[u][i] * scale : -INFINITY;
                mx = fmaxf(mx, sc[u][i]);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));                    // finite: key j0 is inside the split
        const float mn = fmaxf(m, mx);
        const float corr = expf(m - mn);
        m = mn;
        float sum = 0.f;
        #pragma unroll
        for (int u = 0; u < 2; ++u)
        {
            #pragma unroll
            for (int i = 0; i < 4; ++i) { sc[u][i] = expf(sc[u][i] - mn); sum += sc[u][i]; }       // masked: exp(-inf) = 0
        }
        l = l * corr + sum;
        bf16x8 pb;
        #pragma unroll
        for (int i = 0; i < 4; ++i) { pb[i] = (__bf16) sc[0][i]; pb[4 + i] = (__bf16) sc[1][i]; }
        #pragma unroll
        for (int t = 0; t < NVW; ++t)
        {
            acc[t] *= corr;
            const uint16_t* vr = vt + ((w * NVW + t) * 16 + c) * LM_VS;
            union { bf16x8 v; bf16x4 h[2]; } va;
            va.h[0] = *(const bf16x4*) (vr + g * 4);
            va.h[1] = *(const bf16x4*) (vr + 16 + g * 4);
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va.v, pb, acc[t], 0, 0, 0);
        }
    }
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (!head_ok) return;
    if (w == 0 && g == 0) { part_ml[pidx * 2] = m; part_ml[pidx * 2 + 1] = l; }
    float* po = part_o + pidx * (NV * 16) + w * NVW * 16;
    #pragma unroll
    for (int t = 0; t < NVW; ++t) *(f32x4*) (po + t * 16 + g * 4) = acc[t];          // acc[t][i] = latent column (w NVW + t) * 16 + 4g + i of head c
}

// o_lat[n][h] = sum_s e^(m_s - M) O_s / (sum_s e^(m_s - M) l_s + e^(sink - M)), M = max(m_s, sink); splits without keys weigh nothing (their sums are
// never read into the result: unwritten scratch may hold anything).  The splits' weights are computed once into LDS; the sum over splits then has
// independent loads.
__global__ __launch_bounds__(128) void latent_decode_merge_kernel(bf16_t* __restrict__ o_lat, int64_t o_row, int64_t o_head, const float* __restrict__ part_o,
                                                                  const float* __restrict__ part_ml, const float* __restrict__ sink, int splits, int heads, int rank, int rp)
{
    extern __shared__ float wsm[];                              // [splits]
    __shared__ float red[2];
    const int n = blockIdx.x, h = blockIdx.y;
    const float* ml = part_ml + ((int64_t) n * splits * heads + h) * 2;         // split s at ml + s * heads * 2
    const float* po = part_o + ((int64_t) n * splits * heads + h) * rp;         // split s at po + s * heads * rp
    const float sk = sink ? sink[h] : -INFINITY;
    float mloc = -INFINITY;
    for (int s = threadIdx.x; s < splits; s += 128) mloc = fmaxf(mloc, ml[(int64_t) s * heads * 2]);
    mloc = wave_max(mloc);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mloc;
    __syncthreads();
    const float M = fmaxf(fmaxf(red[0], red[1]), sk);
    float lloc = 0.f;
    for (int s = threadIdx.x; s < splits; s += 128)
    {
        const float ls = ml[(int64_t) s * heads * 2 + 1];
        const float w = ls > 0.f ? expf(ml[(int64_t) s * heads * 2] - M) : 0.f;
        wsm[s] = w;
        lloc += w * ls;
    }
    lloc = block_sum<2>(lloc, red);                             // its barriers also publish wsm
    const float L = lloc + (sink ? expf(sk - M) : 0.f);
    const float inv = L > 0.f ? 1.0f / L : 0.f;
    for (int col = threadIdx.x; col < rank; col += 128)
    {
        float a = 0.f;
        #pragma unroll 8
        for (int s = 0; s < splits; ++s)
        {
            const float w = wsm[s], v = po[(int64_t) s * heads * rp + col];
            a += w != 0.f ? w * v : 0.f;
        }
        o_lat[(int64_t) n * o_row + (int64_t) h * o_head + col] = from_f<bf16_t>(a * inv);
    }
}

extern "C" int exl3_mix_latent_decode_mfma_scratch(int n, int heads, int rank, int splits, int64_t* floats)
{
    MIX_CHECK(floats && n >= 0 && heads > 0 && rank > 0 && rank <= 512 && splits > 0, "mix_latent_decode_mfma_scratch: bad arguments");
    const int rp = rank <= 128 ? 128 : (rank <= 256 ? 256 : 512);
    *floats = (int64_t) n * splits * heads * (rp + 2);
    return EXL3_MIX_OK;
}

extern "C" int exl3_mix_latent_decode_mfma(void* o_lat, int64_t o_row, int64_t o_head, const void* q_lat, int64_t ql_row, int64_t ql_head, const void* q, int64_t q_ld,
                                           const void* ring, const float* sink, const int32_t* slots, const int32_t* len_after, float* scratch, int splits,
                                           int n, int heads, int dim, int rot_dim, int rank, float scale, int window, void* stream)
{
    MIX_CHECK(o_lat && q_lat && q && ring && slots && len_after && scratch, "mix_latent_decode_mfma: null pointer");
    MIX_CHECK(n >= 0 && n <= 65535 && heads > 0 && dim >= 0 && window > 0 && splits > 0 && splits <= 65535, "mix_latent_decode_mfma: bad sizes");
    MIX_CHECK(rank > 0 && rank <= 512 && rank % 8 == 0 && rot_dim >= 0 && rot_dim % 8 == 0, "mix_latent_decode_mfma: rank %d and rot_dim %d must be multiples of 8, rank <= 512", rank, rot_dim);
    const int nv = rank <= 128 ? 8 : (rank <= 256 ? 16 : 32);
    MIX_CHECK(rank + rot_dim <= (nv / 2 + LM_WAVES) * 32, "mix_latent_decode_mfma: rot_dim %d too large beside rank %d", rot_dim, rank);
    MIX_CHECK((uintptr_t) ring % 16 == 0 && q_ld >= (int64_t) heads * (dim + rot_dim), "mix_latent_decode_mfma: the ring must be 16-byte aligned");
    if (n == 0) return EXL3_MIX_OK;
    const int keys_per_split = (((window + splits - 1) / splits) + LM_KEYS - 1) / LM_KEYS * LM_KEYS;
    const int rp = nv * 16;
    const int q_vec = (uintptr_t) q_lat % 16 == 0 && ql_row % 8 == 0 && ql_head % 8 == 0 && (uintptr_t) q % 16 == 0 && q_ld % 8 == 0 && dim % 8 == 0;
    float* part_o = scratch;
    float* part_ml = scratch + (int64_t) n * splits * heads * rp;
    const dim3 grid(splits, (heads + 15) / 16, n);
    #define LM_LAUNCH(NVV) hipLaunchKernelGGL((latent_decode_mfma_kernel<NVV>), grid, dim3(64 * LM_WAVES), 0, (hipStream_t) stream, part_o, part_ml, (const bf16_t*) q_lat, ql_row, \
                                              ql_head, (const bf16_t*) q, q_ld, (const bf16_t*) ring, slots, len_after, heads, dim, rot_dim, rank, scale, window, keys_per_split, q_vec)
    if (nv == 8) LM_LAUNCH(8); else if (nv == 16) LM_LAUNCH(16); else LM_LAUNCH(32);
    #undef LM_LAUNCH
    if (int rc = mix_check_launch("mix_latent_decode_mfma")) return rc;
    hipLaunchKernelGGL(latent_decode_merge_kernel, dim3(n, heads), dim3(128), (size_t) splits * sizeof(float), (hipStream_t) stream, (bf16_t*) o_lat, o_row, o_head, part_o, part_ml, sink, splits, heads, rank, rp);
    return mix_check_launch("mix_latent_decode_mfma (merge)");
}
