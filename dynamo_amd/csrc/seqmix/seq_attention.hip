// Softmax attention over the paged cache with a logarithmic distance bias
// and a position-dependent query temperature, for head sizes the MFMA
// flash kernels do not cover (any dk, dv up to 64 * EVMAX) and for fp32
// caches. One wave per (token row, query head): lanes own keys for the
// score pass and value channels for the weighted sum. Scores, softmax and
// the accumulator are fp32.
//
//   score(i, j) = temp(i) * scale * (q_i . k_j) - r1_h * log1p(r2_h * (i - j))
//   temp(i)     = 1 + coef * ln(floor((i + 1) / every) + 1)
//
// The same kernel serves prompt portions and decoded tokens: a row only
// needs its position and its sequence's page table.
#include "seq_common.h"

namespace {

constexpr int EVMAX = 8;  // value channels per lane: dv <= 512

// Append this step's keys (raw) and values (each head divided by its root
// mean square when vnorm is set) to the paged cache. One wave per
// (token, kv head). Cache layout [pages, G, page_size, d].
template <typename T>
__global__ void kv_append_norm_kernel(
    T* __restrict__ kcache, T* __restrict__ vcache, const T* __restrict__ proj,
    int proj_stride, int off_k, int off_v,
    const int64_t* __restrict__ slot_mapping, int G, int dk, int dv, int ps,
    int vnorm, float eps) {
  const int t = blockIdx.x, g = blockIdx.y, lane = threadIdx.x;
  const int64_t slot = slot_mapping[t];
  if (slot < 0) return;
  const int64_t page = slot / ps, inpage = slot % ps;
  const T* krow = proj + (int64_t)t * proj_stride + off_k + g * dk;
  const T* vrow = proj + (int64_t)t * proj_stride + off_v + g * dv;
  T* kd = kcache + ((page * G + g) * ps + inpage) * dk;
  T* vd = vcache + ((page * G + g) * ps + inpage) * dv;
  for (int i = lane; i < dk; i += 64) kd[i] = krow[i];
  float inv = 1.f;
  if (vnorm) {
    float ss = 0.f;
    for (int i = lane; i < dv; i += 64) {
      const float x = to_f(vrow[i]);
      ss += x * x;
    }
    ss = wave_sum(ss);
    inv = 1.f / sqrtf(ss / (float)dv + eps);
  }
  for (int i = lane; i < dv; i += 64) vd[i] = from_f<T>(to_f(vrow[i]) * inv);
}

template <typename T>
__global__ void biased_attention_kernel(
    T* __restrict__ out,  // [T, H, dv]
    const T* __restrict__ proj, int proj_stride, int off_q,
    const T* __restrict__ kcache, const T* __restrict__ vcache,
    const int* __restrict__ page_table, int table_stride,
    const int* __restrict__ tok_seq, const int* __restrict__ positions,
    const int* __restrict__ seq_len, const float* __restrict__ r1,
    const float* __restrict__ r2, int H, int G, int dk, int dv, int ps,
    float scale, float temp_coef, int temp_every, int has_bias) {
  extern __shared__ float qs[];  // [dk] scaled query
  const int t = blockIdx.x, hh = blockIdx.y, lane = threadIdx.x;
  const int s = tok_seq[t];
  if (seq_len[s] == 0) return;  // padding row
  const int pos = positions[t];
  const int g = hh / (H / G);
  float temp = 1.f;
  if (temp_coef != 0.f)
    temp += temp_coef * logf((float)((pos + 1) / temp_every) + 1.f);
  const float qmul = temp * scale;
  const T* q = proj + (int64_t)t * proj_stride + off_q + hh * dk;
  for (int i = lane; i < dk; i += 64) qs[i] = to_f(q[i]) * qmul;
  __syncthreads();
  const int* table = page_table + (int64_t)s * table_stride;
  const float b1 = has_bias ? r1[hh] : 0.f;
  const float b2 = has_bias ? r2[hh] : 0.f;

  float m = -INFINITY, l = 0.f;
  float acc[EVMAX];
#pragma unroll
  for (int e = 0; e < EVMAX; e++) acc[e] = 0.f;
  const int ctx = pos + 1;
  for (int j0 = 0; j0 < ctx; j0 += 64) {
    const int j = j0 + lane;
    float sc = -INFINITY;
    if (j < ctx) {
      const int64_t page = table[j / ps];
      const T* k = kcache + ((page * G + g) * ps + (j % ps)) * dk;
      float d = 0.f;
      for (int i = 0; i < dk; i++) d += qs[i] * to_f(k[i]);
      sc = d;
      if (has_bias) sc -= b1 * log1pf(b2 * (float)(pos - j));
    }
    const float mn = fmaxf(m, wave_max(sc));
    const float corr = expf(m - mn);  // 0 on the first chunk (m = -inf)
    const float p = (j < ctx) ? expf(sc - mn) : 0.f;
    l = l * corr + wave_sum(p);
    m = mn;
#pragma unroll
    for (int e = 0; e < EVMAX; e++) acc[e] *= corr;
    const int n = min(64, ctx - j0);
    for (int jj = 0; jj < n; jj++) {
      const float pj = __shfl(p, jj, 64);
      const int jk = j0 + jj;
      const int64_t page = table[jk / ps];
      const T* v = vcache + ((page * G + g) * ps + (jk % ps)) * dv;
#pragma unroll
      for (int e = 0; e < EVMAX; e++) {
        const int c = lane + 64 * e;
        if (c < dv) acc[e] += pj * to_f(v[c]);
      }
    }
  }
  const float inv = 1.f / l;
#pragma unroll
  for (int e = 0; e < EVMAX; e++) {
    const int c = lane + 64 * e;
    if (c < dv) out[((int64_t)t * H + hh) * dv + c] = from_f<T>(acc[e] * inv);
  }
}

}  // namespace

void kv_append_norm(torch::Tensor kcache, torch::Tensor vcache,
                    torch::Tensor proj, int64_t off_k, int64_t off_v,
                    torch::Tensor slot_mapping, bool vnorm, double eps) {
  // caches [pages, G, ps, d]
  const int T_ = proj.size(0);
  const int G = kcache.size(1), ps = kcache.size(2), dk = kcache.size(3);
  const int dv = vcache.size(3);
  SEQ_CHECK(kcache.is_contiguous() && vcache.is_contiguous() &&
                vcache.size(0) == kcache.size(0) && vcache.size(1) == G &&
                vcache.size(2) == ps &&
                kcache.scalar_type() == proj.scalar_type() &&
                vcache.scalar_type() == proj.scalar_type(), "kv cache");
  SEQ_CHECK(proj.stride(1) == 1 && off_k + G * dk <= proj.size(1) &&
                off_v + G * dv <= proj.size(1), "kv projections");
  SEQ_CHECK(slot_mapping.scalar_type() == torch::kLong &&
                slot_mapping.is_contiguous() && slot_mapping.numel() >= T_,
            "slot mapping");
  if (T_ == 0) return;
  DISPATCH_ACT(proj, hipLaunchKernelGGL(
      kv_append_norm_kernel<T>, dim3(T_, G), dim3(64), 0, cur_stream(),
      ptr<T>(kcache), ptr<T>(vcache), cptr<T>(proj), (int)proj.stride(0),
      (int)off_k, (int)off_v, cptr<int64_t>(slot_mapping), G, dk, dv, ps,
      vnorm ? 1 : 0, (float)eps););
}

void biased_attention(torch::Tensor out, torch::Tensor proj, int64_t off_q,
                      torch::Tensor kcache, torch::Tensor vcache,
                      torch::Tensor page_table, torch::Tensor tok_seq,
                      torch::Tensor positions, torch::Tensor seq_len,
                      c10::optional<torch::Tensor> r1,
                      c10::optional<torch::Tensor> r2, double scale,
                      double temp_coef, int64_t temp_every) {
  const int T_ = out.size(0), H = out.size(1), dv = out.size(2);
  const int G = kcache.size(1), ps = kcache.size(2), dk = kcache.size(3);
  SEQ_CHECK(out.is_contiguous() && out.scalar_type() == proj.scalar_type(),
            "attention out");
  SEQ_CHECK(kcache.is_contiguous() && vcache.is_contiguous() &&
                vcache.size(3) == dv && vcache.size(1) == G &&
                kcache.scalar_type() == proj.scalar_type() &&
                vcache.scalar_type() == proj.scalar_type(), "attention cache");
  SEQ_CHECK(H % G == 0 && dv <= 64 * EVMAX, "attention head sizes");
  SEQ_CHECK(proj.stride(1) == 1 && proj.size(0) == T_ &&
                off_q + H * dk <= proj.size(1), "attention q");
  SEQ_CHECK(page_table.scalar_type() == torch::kInt && page_table.dim() == 2 &&
                page_table.stride(1) == 1, "page table");
  for (const torch::Tensor* t : {&tok_seq, &positions})
    SEQ_CHECK(t->scalar_type() == torch::kInt && t->is_contiguous() &&
                  t->numel() >= T_, "token descriptors");
  SEQ_CHECK(seq_len.scalar_type() == torch::kInt &&
                seq_len.is_contiguous() &&
                seq_len.numel() <= page_table.size(0), "seq_len");
  SEQ_CHECK(r1.has_value() == r2.has_value(), "bias parameters");
  if (r1)
    SEQ_CHECK(r1->scalar_type() == torch::kFloat && r1->numel() == H &&
                  r2->scalar_type() == torch::kFloat && r2->numel() == H,
              "bias parameters");
  SEQ_CHECK(temp_every >= 1, "temperature period");
  if (T_ == 0) return;
  DISPATCH_ACT(proj, hipLaunchKernelGGL(
      biased_attention_kernel<T>, dim3(T_, H), dim3(64), dk * sizeof(float),
      cur_stream(), ptr<T>(out), cptr<T>(proj), (int)proj.stride(0),
      (int)off_q, cptr<T>(kcache), cptr<T>(vcache), cptr<int>(page_table),
      (int)page_table.stride(0), cptr<int>(tok_seq), cptr<int>(positions),
      cptr<int>(seq_len), r1 ? cptr<float>(*r1) : nullptr,
      r2 ? cptr<float>(*r2) : nullptr, H, G, dk, dv, ps, (float)scale,
      (float)temp_coef, (int)temp_every, r1 ? 1 : 0););
}
