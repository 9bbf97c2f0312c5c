// Gated linear attention: a per-head matrix state S [dim, vdim] in fp32 with a data-dependent decay per key channel,
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,   a_t = sigmoid(z_t)^(1/tau),
// followed, in the same launch, by the RMS norm of o_t over vdim (one weight shared by the heads) and the SiLU output
// gate.  One workgroup owns one (request, head) pair and walks the request's tokens of this step in order, starting
// from the request's state slot (or from zero when the request has no tokens behind it) and leaving the state there:
// a prompt portion, the next portion and single decoded tokens all go through this one kernel.
//
// Two kernels: gla_col_kernel (key sizes up to 128: one state column per thread, see there) and gla_kernel for wider
// states, where thread (part, v) keeps the state entries S[part + parts * i][v], i < DPT, in registers and the o_t
// column sums over the parts go through LDS.  The decay is evaluated as exp(log(sigmoid(z)) / tau) with log(sigmoid) in its stable form.
#include "anyt.h"

namespace {

struct GlaArgs {
  const float* proj;     // [tokens, proj_rs]: q | k | v | g at the given column offsets (fp32 projections)
  int64_t proj_rs;
  int q_off, k_off, v_off, g_off;
  const float* z;        // [tokens, z_rs]: decay logits per (head, key channel), bias included
  int64_t z_rs;
  float* state;          // [slots, H, dim, vdim]
  const int32_t* cu_q;   // [B + 1] token ranges of the requests in this step
  const int32_t* past;   // [B] tokens each request already holds
  const int32_t* slots;  // [B] state slot of each request
  const void* norm_w;    // [vdim]
  void* out;             // [tokens, H * vdim]
  int H, dim, vdim, parts;
  float inv_tau, q_scale, eps;
};

template <typename T, int DPT>
__global__ __launch_bounds__(1024) void gla_kernel(GlaArgs p) {
  extern __shared__ float lds[];
  float* sa = lds;                 // [dim] decay
  float* sk = sa + p.dim;          // [dim]
  float* sq = sk + p.dim;          // [dim]
  float* so = sq + p.dim;          // [parts][vdim]
  float* red = so + p.parts * p.vdim;   // [32]
  const int h = blockIdx.x, b = blockIdx.y;
  const int tid = threadIdx.x;
  const bool active = tid < p.parts * p.vdim;
  const int v = tid % p.vdim, part = tid / p.vdim;
  const int t0 = p.cu_q[b], t1 = p.cu_q[b + 1];
  float* S_g = p.state + ((int64_t)p.slots[b] * p.H + h) * p.dim * p.vdim;
  float S[DPT];
  const bool fresh = p.past[b] == 0;
#pragma unroll
  for (int i = 0; i < DPT; ++i) {
    const int d = part + p.parts * i;
    S[i] = (active && d < p.dim && !fresh) ? S_g[(int64_t)d * p.vdim + v] : 0.0f;
  }
  const float nw = active ? ld_f32<T>(reinterpret_cast<const T*>(p.norm_w) + v) : 0.0f;
  for (int t = t0; t < t1; ++t) {
    const float* row = p.proj + (int64_t)t * p.proj_rs;
    for (int j = tid; j < p.dim; j += blockDim.x) {
      sa[j] = expf(log_sigmoid_f32(p.z[(int64_t)t * p.z_rs + h * p.dim + j]) * p.inv_tau);
      sk[j] = row[p.k_off + h * p.dim + j];
      sq[j] = row[p.q_off + h * p.dim + j] * p.q_scale;
    }
    const float vv = active ? row[p.v_off + h * p.vdim + v] : 0.0f;
    __syncthreads();
    float o = 0.0f;
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
      const int d = part + p.parts * i;
      if (d < p.dim) {
        S[i] = sa[d] * S[i] + sk[d] * vv;
        o += S[i] * sq[d];
      }
    }
    if (active) so[part * p.vdim + v] = o;
    __syncthreads();
    float ov = 0.0f;
    if (tid < p.vdim)
      for (int q = 0; q < p.parts; ++q) ov += so[q * p.vdim + tid];
    const float ss = block_sum(tid < p.vdim ? ov * ov : 0.0f, red);
    if (tid < p.vdim) {
      const float inv = 1.0f / sqrtf(ss / (float)p.vdim + p.eps);
      const float gate = row[p.g_off + h * p.vdim + tid];
      st_f32<T>(reinterpret_cast<T*>(p.out) + (int64_t)t * p.H * p.vdim + h * p.vdim + tid,
                ov * inv * nw * silu_f32(gate));
    }
    __syncthreads();   // sa/sk/sq/so are rewritten by the next token
  }
  if (active && t1 > t0) {
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
      const int d = part + p.parts * i;
      if (d < p.dim) S_g[(int64_t)d * p.vdim + v] = S[i];
    }
  }
}


// The usual shape (dim <= 128): thread v owns the whole state column S[:, v] in registers, so o_t[v] needs no sum
// across threads.  Tokens are staged sixteen at a time: decay, k and q rows in LDS (padded to DMAX with a = 1,
// k = q = 0), the thread's own v and gate values in registers; the per-token loop then only reads LDS broadcasts, four
// channels per read; the RMS norm's sum over vdim is taken for the sixteen tokens at once (three barriers per chunk).
constexpr int GLA_TC = 16;

constexpr int gla_col_threads(int per_thread) { return per_thread >= 64 ? 256 : 512; }   // by state registers per thread

template <typename T, int DMAX, int CS>
__global__ __launch_bounds__(gla_col_threads(DMAX / CS)) void gla_col_kernel(GlaArgs p) {
  // CS: the key channels of a column are split over CS threads (more wavefronts per (request, head), shorter per-token
  // chains); their partial o_t meet in LDS once per chunk of tokens.  vdp = threads per split, whole wavefronts.
  constexpr int DC = DMAX / CS;
  extern __shared__ float4 lds4[];
  float* lds = reinterpret_cast<float*>(lds4);
  const int vd = p.vdim;
  const int tid = threadIdx.x, nthr = blockDim.x, vdp = nthr / CS;
  float* sa = lds;                       // [TC][DMAX]
  float* sk = sa + GLA_TC * DMAX;
  float* sq = sk + GLA_TC * DMAX;
  float* sred = sq + GLA_TC * DMAX;      // [TC][waves of one split]
  float* so = sred + GLA_TC * (vdp >> 6);   // [CS][TC][vdp] partial outputs (CS > 1)
  const int h = blockIdx.x, b = blockIdx.y;
  const int v = tid % vdp, cs = tid / vdp, wv = v >> 6, nw = vdp >> 6;
  const int cb = cs * DC;
  const bool active = v < vd;
  const int col = active ? v : 0;
  const int t0 = p.cu_q[b], t1 = p.cu_q[b + 1];
  if (t1 <= t0) return;
  float* S_g = p.state + ((int64_t)p.slots[b] * p.H + h) * p.dim * vd;
  float S[DC];
  const bool fresh = p.past[b] == 0;
#pragma unroll
  for (int i = 0; i < DC; ++i) S[i] = (active && cb + i < p.dim && !fresh) ? S_g[(int64_t)(cb + i) * vd + v] : 0.0f;
  const float nw_v = active ? ld_f32<T>(reinterpret_cast<const T*>(p.norm_w) + v) : 0.0f;
  for (int c0 = t0; c0 < t1; c0 += GLA_TC) {
    const int nt = min(GLA_TC, t1 - c0);
    // this thread's own v and gate values of the chunk: sixteen loads in flight, no LDS
    float vreg[GLA_TC], greg[GLA_TC];
#pragma unroll
    for (int j = 0; j < GLA_TC; ++j) {
      vreg[j] = greg[j] = 0.0f;
      if (j < nt) {
        const float* row = p.proj + (int64_t)(c0 + j) * p.proj_rs;
        vreg[j] = row[p.v_off + h * vd + col];
        if (cs == 0) greg[j] = row[p.g_off + h * vd + col];
      }
    }
    __syncthreads();                     // the previous chunk's rows are no longer read
    // decay, k and q rows of the chunk, four elements per thread and step so that the loads overlap
    for (int base = tid * 4; base < nt * DMAX; base += nthr * 4) {
      const int j = base / DMAX, i = base % DMAX;          // DMAX is a multiple of 4: the four share a token
      float z4[4], k4[4], q4[4];
      const float* row = p.proj + (int64_t)(c0 + j) * p.proj_rs;
      const float* zr = p.z + (int64_t)(c0 + j) * p.z_rs;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool in = i + e < p.dim;
        const int ch = h * p.dim + (in ? i + e : 0);
        z4[e] = zr[ch];
        k4[e] = in ? row[p.k_off + ch] : 0.0f;
        q4[e] = in ? row[p.q_off + ch] * p.q_scale : 0.0f;
        z4[e] = in ? expf(log_sigmoid_f32(z4[e]) * p.inv_tau) : 1.0f;
      }
      *reinterpret_cast<float4*>(sa + base) = make_float4(z4[0], z4[1], z4[2], z4[3]);
      *reinterpret_cast<float4*>(sk + base) = make_float4(k4[0], k4[1], k4[2], k4[3]);
      *reinterpret_cast<float4*>(sq + base) = make_float4(q4[0], q4[1], q4[2], q4[3]);
    }
    __syncthreads();
    float o[GLA_TC];
#pragma unroll
    for (int j = 0; j < GLA_TC; ++j) {
      float acc0 = 0.0f, acc1 = 0.0f;
      if (j < nt) {
        const float vv = vreg[j];
        const float4* a4 = reinterpret_cast<const float4*>(sa + j * DMAX + cb);
        const float4* k4 = reinterpret_cast<const float4*>(sk + j * DMAX + cb);
        const float4* q4 = reinterpret_cast<const float4*>(sq + j * DMAX + cb);
#pragma unroll
        for (int i = 0; i < DC / 4; ++i) {
          const float4 a = a4[i], k = k4[i], q = q4[i];
          S[4 * i + 0] = a.x * S[4 * i + 0] + k.x * vv;
          S[4 * i + 1] = a.y * S[4 * i + 1] + k.y * vv;
          S[4 * i + 2] = a.z * S[4 * i + 2] + k.z * vv;
          S[4 * i + 3] = a.w * S[4 * i + 3] + k.w * vv;
          acc0 += S[4 * i + 0] * q.x;
          acc1 += S[4 * i + 1] * q.y;
          acc0 += S[4 * i + 2] * q.z;
          acc1 += S[4 * i + 3] * q.w;
        }
      }
      o[j] = acc0 + acc1;
    }
    if constexpr (CS > 1) {
#pragma unroll
      for (int j = 0; j < GLA_TC; ++j) so[(cs * GLA_TC + j) * vdp + v] = o[j];
      __syncthreads();
    }
    if (cs == 0) {
#pragma unroll
      for (int j = 0; j < GLA_TC; ++j) {
        if constexpr (CS > 1) {
          float t = 0.0f;
#pragma unroll
          for (int q = 0; q < CS; ++q) t += so[(q * GLA_TC + j) * vdp + v];
          o[j] = t;
        }
        const float ss = wave_sum(active ? o[j] * o[j] : 0.0f);
        if ((tid & 63) == 0) sred[j * nw + wv] = ss;
      }
    }
    __syncthreads();
    if (cs == 0 && active) {
#pragma unroll
      for (int j = 0; j < GLA_TC; ++j) {
        if (j < nt) {
          float ss = 0.0f;
          for (int w = 0; w < nw; ++w) ss += sred[j * nw + w];
          const float inv = 1.0f / sqrtf(ss / (float)vd + p.eps);
          st_f32<T>(reinterpret_cast<T*>(p.out) + (int64_t)(c0 + j) * p.H * vd + h * vd + v,
                    o[j] * inv * nw_v * silu_f32(greg[j]));
        }
      }
    }
  }
  if (active) {
#pragma unroll
    for (int i = 0; i < DC; ++i)
      if (cb + i < p.dim) S_g[(int64_t)(cb + i) * vd + v] = S[i];
  }
}

template <typename T, int DMAX>
int launch_col_cs(const GlaArgs& p, int cs, dim3 grid, int threads, size_t lds, hipStream_t s) {
  if (cs == 4) gla_col_kernel<T, DMAX, 4><<<grid, dim3(threads), lds, s>>>(p);
  else if (cs == 2) gla_col_kernel<T, DMAX, 2><<<grid, dim3(threads), lds, s>>>(p);
  else gla_col_kernel<T, DMAX, 1><<<grid, dim3(threads), lds, s>>>(p);
  return 0;
}

template <typename T>
int launch_col(const GlaArgs& p, int dmax, int cs, dim3 grid, int threads, size_t lds, hipStream_t s) {
  switch (dmax) {
    case 16: return launch_col_cs<T, 16>(p, cs, grid, threads, lds, s);
    case 32: return launch_col_cs<T, 32>(p, cs, grid, threads, lds, s);
    case 64: return launch_col_cs<T, 64>(p, cs, grid, threads, lds, s);
    default: return launch_col_cs<T, 128>(p, cs, grid, threads, lds, s);
  }
}

template <typename T>
int launch(const GlaArgs& p, int dpt, dim3 grid, int threads, size_t lds, hipStream_t s) {
  switch (dpt) {
    case 8: gla_kernel<T, 8><<<grid, dim3(threads), lds, s>>>(p); break;
    case 16: gla_kernel<T, 16><<<grid, dim3(threads), lds, s>>>(p); break;
    case 32: gla_kernel<T, 32><<<grid, dim3(threads), lds, s>>>(p); break;
    default: gla_kernel<T, 64><<<grid, dim3(threads), lds, s>>>(p); break;
  }
  return 0;
}

}  // namespace

extern "C" int nv_gla_recurrent(const float* proj, int64_t proj_row_stride, int q_off, int k_off, int v_off, int g_off,
                                const float* z, int64_t z_row_stride, float* state, const int32_t* cu_q,
                                const int32_t* past_lens, const int32_t* state_slots, const void* norm_w, void* out,
                                int num_seqs, int heads, int dim, int vdim, float tau, float q_scale, float eps,
                                int dtype, nv_stream_t stream) {
  NV_CHECK_ARG(proj && z && state && cu_q && past_lens && state_slots && norm_w && out, "nv_gla_recurrent: null pointer");
  NV_CHECK_ARG(dtype == NV_BF16 || dtype == NV_F32, "nv_gla_recurrent: bad dtype %d", dtype);
  NV_CHECK_ARG(heads > 0 && heads <= 65535 && dim > 0 && vdim > 0 && vdim <= 1024 && num_seqs >= 0 && num_seqs <= 65535,
               "nv_gla_recurrent: bad shape heads=%d dim=%d vdim=%d seqs=%d", heads, dim, vdim, num_seqs);
  NV_CHECK_ARG(tau > 0.0f, "nv_gla_recurrent: tau must be positive");
  if (num_seqs == 0) return NV_OK;
  if (dim <= 128) {     // one state column per thread (or per CS threads)
    int dmax = 16;
    while (dmax < dim) dmax *= 2;
    const int vdp = ((vdim + 63) / 64) * 64;
    int cs = 1;
    while (cs < 4 && vdp * cs * 2 <= 256 && dmax / (cs * 2) >= 16) cs *= 2;
    const int threads = vdp * cs;
    const size_t lds = (size_t)(GLA_TC * 3 * dmax + GLA_TC * (vdp / 64) + (cs > 1 ? cs * GLA_TC * vdp : 0)) * sizeof(float);
    if (lds <= 64 * 1024 && threads <= gla_col_threads(dmax / cs)) {
      GlaArgs p{proj, proj_row_stride, q_off, k_off, v_off, g_off, z, z_row_stride, state, cu_q, past_lens, state_slots,
                norm_w, out, heads, dim, vdim, 1, 1.0f / tau, q_scale, eps};
      NV_DISPATCH_T(dtype, launch_col<T>(p, dmax, cs, dim3(heads, num_seqs), threads, lds, (hipStream_t)stream));
      NV_CHECK_LAUNCH();
      return NV_OK;
    }
  }
  int dpt = 8;
  while (dpt <= 64 && ((dim + dpt - 1) / dpt) * vdim > 1024) dpt *= 2;
  if (dpt > 64) {
    nv_set_error("nv_gla_recurrent: a %d x %d state does not fit one workgroup's registers", dim, vdim);
    return NV_ERR_UNSUPPORTED;
  }
  GlaArgs p{proj, proj_row_stride, q_off, k_off, v_off, g_off, z, z_row_stride, state, cu_q, past_lens, state_slots,
            norm_w, out, heads, dim, vdim, (dim + dpt - 1) / dpt, 1.0f / tau, q_scale, eps};
  int threads = ((p.parts * vdim + 63) / 64) * 64;
  const size_t lds = (size_t)(3 * dim + p.parts * vdim + 32) * sizeof(float);
  NV_CHECK_ARG(lds <= 64 * 1024, "nv_gla_recurrent: dim=%d needs %zu bytes of LDS", dim, lds);
  dim3 grid(heads, num_seqs);
  NV_DISPATCH_T(dtype, launch<T>(p, dpt, grid, threads, lds, (hipStream_t)stream));
  NV_CHECK_LAUNCH();
  return NV_OK;
}
