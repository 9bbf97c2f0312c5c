// Gated linear attention: a per-head matrix state S [dim, vdim] in fp32 with a data-dependent decay per key channel,
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,   a_t = sigmoid(z_t)^(1/tau),
// followed, in the same launch, by the RMS norm of o_t over vdim (one weight shared by the heads) and the SiLU output
// gate.  One workgroup owns one (request, head) pair and walks the request's tokens of this step in order, starting
// from the request's state slot (or from zero when the request has no tokens behind it) and leaving the state there:
// a prompt portion, the next portion and single decoded tokens all go through this one kernel.
//
// Thread (part, v) keeps the state entries S[part + parts * i][v], i < DPT, in registers; the o_t column sums over the
// parts go through LDS.  The decay is evaluated as exp(log(sigmoid(z)) / tau) with log(sigmoid) in its stable form.
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
