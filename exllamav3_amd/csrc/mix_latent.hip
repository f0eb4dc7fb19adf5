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
    // the shared key part: rotated pairs, then what lies beyond rot_dims unchanged
    for (int i = threadIdx.x; i < pairs; i += 256)
    {
        const float a = p * freq[i];
        const float cs = cosf(a) * mag, sn = sinf(a) * mag;
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
        const float a = p * freq[i];
        const float cs = cosf(a) * mag, sn = sinf(a) * mag;
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
    MIX_DISPATCH_T(dtype, hipLaunchKernelGGL(latent_prep_kernel<T>, dim3(n), dim3(256), 0, (hipStream_t) stream, (T*) ckr, (T*) ring, (const T*) dkv, dkv_ld, norm_w,
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
