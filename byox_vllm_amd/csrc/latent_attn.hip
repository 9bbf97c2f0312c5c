// Latent attention over a paged cache that holds, per token, one row [latent c (kv_rank) | rotated key part (rot_dim)]
// shared by all heads.  Queries arrive in absorbed form: for head h the first kv_rank numbers are W_uk[h]^T q_unrotated
// (so that their product with c equals q_unrotated . (W_uk[h] c)), the last rot_dim are the rotated query part.  The
// kernel returns sum_j p_j c_j per head; the caller applies W_uv[h] afterwards.  Every head of a token reads the same
// key rows, so a workgroup stages a tile of them in LDS once and serves all its heads from it.
//
//   nv_latent_kv_store : RMS norm of the latent, rotation of the shared key part, store into the token's cache row
//   nv_latent_q_rope   : rotation of the per-head query parts into the absorbed-query buffer
//   nv_latent_attn     : sliding-window softmax attention, one workgroup per (token, group of heads)
//
// Rotation ("rotate half"): dimension i pairs with i + dims/2; the angle is position * inv_freq[i] in fp32, and both
// cosine and sine are multiplied by `mscale` (the caller folds frequency scaling into inv_freq and mscale).
#include "anyt.h"

namespace {

template <typename T>
__global__ __launch_bounds__(256) void latent_kv_store_kernel(const float* __restrict__ kv, int64_t kv_rs,
                                                              const T* __restrict__ norm_w,
                                                              const int64_t* __restrict__ positions,
                                                              const float* __restrict__ inv_freq, float mscale,
                                                              const int32_t* __restrict__ slot_mapping,
                                                              T* __restrict__ cache, int rank, int rot_dim, int rot_dims,
                                                              float eps) {
  __shared__ float red[32];
  const int64_t t = blockIdx.x;
  const int32_t slot = slot_mapping[t];
  const float* row = kv + t * kv_rs;
  float ss = 0.0f;
  for (int j = threadIdx.x; j < rank; j += blockDim.x) ss += row[j] * row[j];
  ss = block_sum(ss, red);
  if (slot < 0) return;
  const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
  T* dst = cache + (int64_t)slot * (rank + rot_dim);
  for (int j = threadIdx.x; j < rank; j += blockDim.x) st_f32<T>(dst + j, row[j] * inv * ld_f32<T>(norm_w + j));
  const float pos = (float)positions[t];
  const int half = rot_dims / 2;
  for (int j = threadIdx.x; j < rot_dim; j += blockDim.x) {
    float v = row[rank + j];
    if (j < rot_dims) {
      const int i = j < half ? j : j - half;
      const float a = pos * inv_freq[i];
      const float cs = cosf(a) * mscale, sn = sinf(a) * mscale;
      const float other = row[rank + (j < half ? j + half : j - half)];
      v = j < half ? v * cs - other * sn : v * cs + other * sn;
    }
    st_f32<T>(dst + rank + j, v);
  }
}

// q [tokens, H * (dim + rot_dim)] in storage type -> qa[t, h, rank .. rank + rot_dim) fp32, rotated
template <typename T>
__global__ __launch_bounds__(256) void latent_q_rope_kernel(const T* __restrict__ q, int64_t q_rs,
                                                            const int64_t* __restrict__ positions,
                                                            const float* __restrict__ inv_freq, float mscale,
                                                            float* __restrict__ qa, int H, int dim, int rot_dim,
                                                            int rot_dims, int rank) {
  const int64_t t = blockIdx.x;
  const float pos = (float)positions[t];
  const int half = rot_dims / 2;
  for (int idx = threadIdx.x; idx < H * rot_dim; idx += blockDim.x) {
    const int h = idx / rot_dim, j = idx % rot_dim;
    const T* src = q + t * q_rs + (int64_t)h * (dim + rot_dim) + dim;
    float v = ld_f32<T>(src + j);
    if (j < rot_dims) {
      const int i = j < half ? j : j - half;
      const float a = pos * inv_freq[i];
      const float cs = cosf(a) * mscale, sn = sinf(a) * mscale;
      const float other = ld_f32<T>(src + (j < half ? j + half : j - half));
      v = j < half ? v * cs - other * sn : v * cs + other * sn;
    }
    qa[(t * H + h) * (rank + rot_dim) + rank + j] = v;
  }
}

struct AttnArgs {
  const float* qa;         // [tokens, H, rank + rot_dim]
  const void* cache;       // [rows, rank + rot_dim]
  const int32_t* tables;   // [B, table_cols]
  int table_cols;
  const int32_t* cu_q;     // [B + 1]
  const int32_t* past;     // [B]
  const int32_t* seq_of;   // [tokens] request index of each token
  void* out;               // [tokens, H, rank]
  int H, rank, rot_dim, block_size, window, HC, TK;
  float scale;
};

template <typename T>
__global__ __launch_bounds__(256) void latent_attn_kernel(AttnArgs p) {
  extern __shared__ float lds[];
  const int Dk = p.rank + p.rot_dim, Dp = Dk + 1;
  const int HC = p.HC, TK = p.TK;
  float* sq = lds;                    // [HC][Dk]
  float* skey = sq + HC * Dk;         // [TK][Dp]
  float* sc = skey + TK * Dp;         // [HC][TK]
  float* acc = sc + HC * TK;          // [HC][rank]
  float* sm = acc + HC * p.rank;      // [HC] running maximum
  float* sl = sm + HC;                // [HC] running sum
  float* scorr = sl + HC;             // [HC]
  const int t = blockIdx.y, h0 = blockIdx.x * HC;
  const int nh = min(HC, p.H - h0);
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int b = p.seq_of[t];
  const int pos = p.past[b] + (t - p.cu_q[b]);
  const int lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
  const int32_t* table = p.tables + (int64_t)b * p.table_cols;
  const T* cache = reinterpret_cast<const T*>(p.cache);

  for (int i = tid; i < nh * Dk; i += 256) sq[i] = p.qa[((int64_t)t * p.H + h0) * Dk + i];
  for (int i = tid; i < nh * p.rank; i += 256) acc[i] = 0.0f;
  if (tid < nh) {
    sm[tid] = -INFINITY;
    sl[tid] = 0.0f;
  }
  __syncthreads();
  for (int j0 = lo; j0 <= pos; j0 += TK) {
    const int nk = min(TK, pos + 1 - j0);
    for (int i = tid; i < nk * Dk; i += 256) {
      const int j = i / Dk, e = i % Dk;
      const int kp = j0 + j;
      const int64_t row = (int64_t)table[kp / p.block_size] * p.block_size + kp % p.block_size;
      skey[j * Dp + e] = ld_f32<T>(cache + row * Dk + e);
    }
    __syncthreads();
    for (int i = tid; i < nh * TK; i += 256) {
      const int h = i / TK, j = i % TK;
      float s = -INFINITY;
      if (j < nk) {
        s = 0.0f;
        const float* qv = sq + h * Dk;
        const float* kv = skey + j * Dp;
        for (int e = 0; e < Dk; ++e) s += qv[e] * kv[e];
        s *= p.scale;
      }
      sc[h * TK + j] = s;
    }
    __syncthreads();
    for (int h = wv; h < nh; h += 4) {
      float m = -INFINITY;
      for (int j = lane; j < TK; j += 64) m = fmaxf(m, sc[h * TK + j]);
      m = wave_max(m);
      const float m_old = sm[h];
      const float m_new = fmaxf(m_old, m);
      float sum = 0.0f;
      for (int j = lane; j < TK; j += 64) {
        const float e = (j < nk) ? expf(sc[h * TK + j] - m_new) : 0.0f;
        sc[h * TK + j] = e;
        sum += e;
      }
      sum = wave_sum(sum);
      if (lane == 0) {
        const float corr = expf(m_old - m_new);   // exp(-inf) = 0 at the first tile
        scorr[h] = corr;
        sm[h] = m_new;
        sl[h] = sl[h] * corr + sum;
      }
    }
    __syncthreads();
    for (int i = tid; i < nh * p.rank; i += 256) {
      const int h = i / p.rank, e = i % p.rank;
      float a = acc[i] * scorr[h];
      const float* pv = sc + h * TK;
      for (int j = 0; j < nk; ++j) a += pv[j] * skey[j * Dp + e];
      acc[i] = a;
    }
    __syncthreads();
  }
  T* out = reinterpret_cast<T*>(p.out);
  for (int i = tid; i < nh * p.rank; i += 256) {
    const int h = i / p.rank;
    st_f32<T>(out + ((int64_t)t * p.H + h0) * p.rank + i, acc[i] / sl[h]);
  }
}

}  // namespace

extern "C" int nv_latent_kv_store(const float* kv, int64_t kv_row_stride, const void* norm_w, const int64_t* positions,
                                  const float* inv_freq, float mscale, const int32_t* slot_mapping, void* cache,
                                  int64_t tokens, int rank, int rot_dim, int rot_dims, float eps, int dtype,
                                  nv_stream_t stream) {
  NV_CHECK_ARG(kv && norm_w && positions && inv_freq && slot_mapping && cache, "nv_latent_kv_store: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_latent_kv_store: bad dtype %d", dtype);
  NV_CHECK_ARG(tokens >= 0 && rank > 0 && rot_dim >= 0 && rot_dims >= 0 && rot_dims <= rot_dim && rot_dims % 2 == 0,
               "nv_latent_kv_store: bad shape rank=%d rot_dim=%d rot_dims=%d", rank, rot_dim, rot_dims);
  if (tokens == 0) return NV_OK;
  NV_DISPATCH_T(dtype, latent_kv_store_kernel<T><<<dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream>>>(
                           kv, kv_row_stride, (const T*)norm_w, positions, inv_freq, mscale, slot_mapping, (T*)cache,
                           rank, rot_dim, rot_dims, eps));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_latent_q_rope(const void* q, int64_t q_row_stride, const int64_t* positions, const float* inv_freq,
                                float mscale, float* qa, int64_t tokens, int heads, int dim, int rot_dim, int rot_dims,
                                int rank, int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(q && positions && inv_freq && qa, "nv_latent_q_rope: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_latent_q_rope: bad dtype %d", dtype);
  NV_CHECK_ARG(tokens >= 0 && heads > 0 && dim >= 0 && rot_dim >= 0 && rot_dims <= rot_dim && rot_dims % 2 == 0 && rank > 0,
               "nv_latent_q_rope: bad shape");
  if (tokens == 0 || rot_dim == 0) return NV_OK;
  NV_DISPATCH_T(dtype, latent_q_rope_kernel<T><<<dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream>>>(
                           (const T*)q, q_row_stride, positions, inv_freq, mscale, qa, heads, dim, rot_dim, rot_dims, rank));
  NV_CHECK_LAUNCH();
  return NV_OK;
}

extern "C" int nv_latent_attn(const float* qa, const void* cache, const int32_t* block_tables, int table_cols,
                              const int32_t* cu_q, const int32_t* past_lens, const int32_t* seq_of_token, void* out,
                              int64_t tokens, int heads, int rank, int rot_dim, int block_size, int window, float scale,
                              int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(qa && cache && block_tables && cu_q && past_lens && seq_of_token && out, "nv_latent_attn: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_latent_attn: bad dtype %d", dtype);
  NV_CHECK_ARG(tokens >= 0 && tokens <= 65535 * 1024 && heads > 0 && rank > 0 && rot_dim >= 0 && block_size > 0 && table_cols > 0,
               "nv_latent_attn: bad shape");
  if (tokens == 0) return NV_OK;
  NV_CHECK_ARG(tokens <= 65535, "nv_latent_attn: %lld tokens exceed one launch", (long long)tokens);
  const int Dk = rank + rot_dim;
  // LDS plan: as many heads per workgroup as fit beside a key tile of 64 (then 32, 16, 8) rows
  const size_t budget = 64 * 1024;
  int TK = 64, HC = heads;
  auto need = [&](int hc, int tk) {
    return (size_t)(hc * Dk + tk * (Dk + 1) + hc * tk + hc * rank + 3 * hc) * sizeof(float);
  };
  while (TK > 8 && need(1, TK) > budget) TK /= 2;
  NV_CHECK_ARG(need(1, TK) <= budget, "nv_latent_attn: rows of %d numbers do not fit the LDS plan", Dk);
  while (HC > 1 && need(HC, TK) > budget) HC = (HC + 1) / 2;
  AttnArgs p{qa, cache, block_tables, table_cols, cu_q, past_lens, seq_of_token, out, heads, rank, rot_dim, block_size,
             window, HC, TK, scale};
  dim3 grid((unsigned)((heads + HC - 1) / HC), (unsigned)tokens);
  NV_DISPATCH_T(dtype, latent_attn_kernel<T><<<grid, dim3(256), need(HC, TK), (hipStream_t)stream>>>(p));
  NV_CHECK_LAUNCH();
  return NV_OK;
}
