// Latent attention of the layer-list models: what a token leaves behind is its normalised key-value latent c (kv_rank numbers) and one rotated
// key part shared by all heads (rot_dim numbers), kept in a per-sequence RING of `cap` rows (row = position mod cap; cap >= window - 1 + the
// widest step, so a step never overwrites a row one of its own tokens still sees).  Scores, soft-max and the weighted sum are fp32.
//   latent_prep_kernel   norms of the two latents, rotation of the shared key part, ring append
//   latent_attn_kernel   one wave per (token, head) over per-head keys / values expanded from the ring rows of the window (the plain form)
#include "ps_seq.h"

#include <cmath>

static __device__ __forceinline__ float la_wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
static __device__ __forceinline__ float la_wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

__global__ __launch_bounds__(256) void latent_prep_kernel(const ps_seq_step *step, long long ring_off, int cap, const float *y, long long ldy, const float *qnorm,
                                                          const float *kvnorm, float eps, int q_rank, int kv_rank, int rot_dim, int rot_dims, const float *freq, float *cq,
                                                          long long ldcq) {
    __shared__ float red[8];
    const int t = blockIdx.x, tid = threadIdx.x;
    const long long pos = step->pos0 + t;
    const float *yt = y + (long long)t * ldy, *ckv = yt + q_rank, *kr = ckv + kv_rank;
    float *ring = step->state + ring_off + (pos % cap) * (long long)(kv_rank + rot_dim);
    float a = 0.f, b = 0.f;
    for (int i = tid; i < q_rank; i += 256) a += yt[i] * yt[i];
    for (int i = tid; i < kv_rank; i += 256) b += ckv[i] * ckv[i];
    a = la_wave_sum(a);
    b = la_wave_sum(b);
    if ((tid & 63) == 0) { red[tid >> 6] = a; red[4 + (tid >> 6)] = b; }
    __syncthreads();
    const float ia = 1.f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)q_rank + eps);
    const float ib = 1.f / sqrtf((red[4] + red[5] + red[6] + red[7]) / (float)kv_rank + eps);
    for (int i = tid; i < q_rank; i += 256) cq[(long long)t * ldcq + i] = yt[i] * ia * qnorm[i];
    for (int i = tid; i < kv_rank; i += 256) ring[i] = ckv[i] * ib * kvnorm[i];
    const int half = rot_dims / 2; // the first rot_dims of the part are rotated, pairs (i, i + rot_dims / 2); the rest passes unchanged
    for (int i = tid; i < half; i += 256) {
        const float ang = (float)pos * freq[i], c = cosf(ang), s = sinf(ang);
        const float u = kr[i], v = kr[i + half];
        ring[kv_rank + i] = u * c - v * s;
        ring[kv_rank + half + i] = v * c + u * s;
    }
    for (int i = 2 * half + tid; i < rot_dim; i += 256) ring[kv_rank + i] = kr[i];
}
void psk_latent_prep(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, const float *y, int64_t ldy, const float *qnorm, const float *kvnorm,
                     float eps, int q_rank, int kv_rank, int rot_dim, int rot_dims, const float *freq, int T, float *cq, int64_t ldcq) {
    hipLaunchKernelGGL(latent_prep_kernel, dim3(T), dim3(256), 0, st, step, (long long)ring_off, cap, y, (long long)ldy, qnorm, kvnorm, eps, q_rank, kv_rank, rot_dim,
                       rot_dims, freq, cq, (long long)ldcq);
}

// dynamic LDS: qs [d + dr], ps [64]
#define LA_NV 4 // value columns per lane: dv <= 256
__global__ __launch_bounds__(64) void latent_attn_kernel(const ps_seq_step *step, long long ring_off, int cap, const float *q, long long ldq, const float *kv,
                                                         long long ldkv, const float *freq, int H, int d, int dr, int rot_dims, int dv, int kv_rank, int window,
                                                         float scale, float *o, long long ldo) {
    extern __shared__ float lds[];
    float *qs = lds, *ps = lds + d + dr;
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const long long pos0 = step->pos0, p = pos0 + t;
    const long long first = pos0 - window + 1 > 0 ? pos0 - window + 1 : 0; // position of kv row 0
    const long long lo = p - window + 1 > 0 ? p - window + 1 : 0;
    const float *qt = q + (long long)t * ldq + (long long)h * (d + dr);
    const int half = rot_dims / 2;
    for (int i = lane; i < d; i += 64) qs[i] = qt[i];
    for (int i = 2 * half + lane; i < dr; i += 64) qs[d + i] = qt[d + i];
    for (int i = lane; i < half; i += 64) {
        const float ang = (float)p * freq[i], c = cosf(ang), s = sinf(ang);
        const float u = qt[d + i], v = qt[d + half + i];
        qs[d + i] = u * c - v * s;
        qs[d + half + i] = v * c + u * s;
    }
    __syncthreads();
    const float *ring = step->state + ring_off;
    const long long rs = kv_rank + dr;
    float m = -INFINITY, l = 0.f, acc[LA_NV];
#pragma unroll
    for (int x = 0; x < LA_NV; x++) acc[x] = 0.f;
    for (long long j0 = lo; j0 <= p; j0 += 64) {
        const long long j = j0 + lane;
        float s = -INFINITY;
        if (j <= p) {
            const float *kn = kv + (j - first) * ldkv + (long long)h * d;
            const float *kr = ring + (j % cap) * rs + kv_rank;
            float a = 0.f;
            for (int i = 0; i < d; i++) a = fmaf(qs[i], kn[i], a);
            for (int i = 0; i < dr; i++) a = fmaf(qs[d + i], kr[i], a);
            s = a * scale;
        }
        const float mn = fmaxf(m, la_wave_max(s));
        const float corr = expf(m - mn), pj = j <= p ? expf(s - mn) : 0.f; // (m = -inf in the first round: corr = 0, acc and l are 0)
        l = l * corr + la_wave_sum(pj);
        m = mn;
        __syncthreads();
        ps[lane] = pj;
        __syncthreads();
        const int nk = (int)min((long long)64, p - j0 + 1);
#pragma unroll
        for (int x = 0; x < LA_NV; x++) acc[x] *= corr;
        for (int kk = 0; kk < nk; kk++) {
            const float *vr = kv + (j0 + kk - first) * ldkv + (long long)H * d + (long long)h * dv;
            const float pk = ps[kk];
#pragma unroll
            for (int x = 0; x < LA_NV; x++)
                if (lane + 64 * x < dv) acc[x] = fmaf(pk, vr[lane + 64 * x], acc[x]);
        }
    }
    const float il = 1.f / l;
#pragma unroll
    for (int x = 0; x < LA_NV; x++)
        if (lane + 64 * x < dv) o[(long long)t * ldo + (long long)h * dv + lane + 64 * x] = acc[x] * il;
}
void psk_latent_attn(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, const float *q, int64_t ldq, const float *kv, int64_t ldkv,
                     const float *freq, int H, int d, int dr, int rot_dims, int dv, int kv_rank, int window, float scale, int T, float *o, int64_t ldo) {
    hipLaunchKernelGGL(latent_attn_kernel, dim3(T, H), dim3(64), (size_t)(d + dr + 64) * 4, st, step, (long long)ring_off, cap, q, (long long)ldq, kv, (long long)ldkv,
                       freq, H, d, dr, rot_dims, dv, kv_rank, window, scale, o, (long long)ldo);
}
