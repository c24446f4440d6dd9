// Prompt-portion attention for the distance-biased softmax attention, on the
// matrix cores (bf16 only): scores and the weighted sum are
// mfma_f32_16x16x32_bf16 products, everything between them is fp32.
//
// A workgroup (4 waves) owns a tile of up to 64 consecutive rows of one
// sequence and one query head; each wave owns 16 rows. Keys and values of
// the kv head are walked in blocks of 64: K rows are staged in LDS as they
// lie in the page (zero padded to a multiple of 32 channels), V is staged
// transposed (channel-major) so that the B operand of the second product
// is a 16-byte run of keys. The fp32 scores get the row's temperature and
// scale, the log distance penalty and the causal mask, then an online
// softmax; the weights pass through LDS as a bf16 hi + lo pair to become
// the A operand of two products.
//
// Fragment layouts of mfma_f32_16x16x32_bf16 (lane l, lr = l % 16,
// lg = l / 16):  A: A[row = lr][k = 8 lg + i], i = 0..7
//                B: B[k = 8 lg + i][col = lr]
//                D: D[row = 4 lg + r][col = lr], r = 0..3
#include "seq_common.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) short short8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

constexpr int BN = 64;    // keys per block
constexpr int PADE = 8;   // padding elements per LDS row (16 bytes)

// KC = padded key size / 32, DN = padded value size / 16
template <int KC, int DN>
__global__ __launch_bounds__(256) void biased_attention_mfma_kernel(
    bf16_t* __restrict__ out,  // [T, H, dv]
    const bf16_t* __restrict__ proj, int proj_stride, int off_q,
    const bf16_t* __restrict__ kcache, const bf16_t* __restrict__ vcache,
    const int* __restrict__ page_table, int table_stride,
    const int* __restrict__ tile_row0, const int* __restrict__ tile_rows,
    const int* __restrict__ tok_seq, const int* __restrict__ positions,
    const float* __restrict__ r1, const float* __restrict__ r2, int H, int G,
    int dk, int dv, int ps, float scale, float temp_coef, int temp_every,
    int has_bias) {
  constexpr int DKP = KC * 32, DVP = DN * 16;
  constexpr int KS = DKP + PADE;  // k_lds row stride (elements)
  constexpr int VS = BN + PADE;   // vt_lds / p_lds row stride
  extern __shared__ __attribute__((aligned(16))) short smem[];
  short* k_lds = smem;                  // [BN][KS]
  short* vt_lds = k_lds + BN * KS;      // [DVP][VS]
  short* p_lds = vt_lds + DVP * VS;     // [4][16][VS]

  const int tile = blockIdx.x, h = blockIdx.y;
  const int g = h / (H / G);
  const int row0 = tile_row0[tile], nrows = tile_rows[tile];
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int lr = lane & 15, lg = lane >> 4;
  const int* table = page_table + (int64_t)tok_seq[row0] * table_stride;

  // ---- Q fragments of row wid*16 + lr (zero beyond dk / beyond the tile)
  bf16x8_t q_frag[KC];
  {
    const int arow = wid * 16 + lr;
    const bool ok = arow < nrows;
    const bf16_t* q =
        proj + (int64_t)(row0 + (ok ? arow : 0)) * proj_stride + off_q + h * dk;
#pragma unroll
    for (int kc = 0; kc < KC; kc++) {
      short8_t v;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const int col = kc * 32 + lg * 8 + i;
        v[i] = (ok && col < dk) ? (short)q[col] : (short)0;
      }
      q_frag[kc] = *reinterpret_cast<bf16x8_t*>(&v);
    }
  }
  // ---- the 4 score rows this lane holds: wid*16 + 4 lg + r
  int pos_r[4];
  float qmul[4];
  bool ok_r[4];
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const int cr = wid * 16 + lg * 4 + r;
    ok_r[r] = cr < nrows;
    pos_r[r] = ok_r[r] ? positions[row0 + cr] : 0;  // key 0 always exists
    float temp = 1.f;
    if (temp_coef != 0.f)
      temp += temp_coef * logf((float)((pos_r[r] + 1) / temp_every) + 1.f);
    qmul[r] = temp * scale;
  }
  const float b1 = has_bias ? r1[h] : 0.f;
  const float b2 = has_bias ? r2[h] : 0.f;
  const int kv_end = positions[row0 + nrows - 1] + 1;  // rows are in order

  float m[4], l[4];
  f32x4_t acc_o[DN];
#pragma unroll
  for (int r = 0; r < 4; r++) {
    m[r] = -INFINITY;
    l[r] = 0.f;
  }
#pragma unroll
  for (int d = 0; d < DN; d++) acc_o[d] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const int kvecs = DKP / 8, vvecs = DVP / 8;
  for (int t0 = 0; t0 < kv_end; t0 += BN) {
    __syncthreads();  // the previous block's readers are done
    // ---- stage K [BN][DKP] and V^T [DVP][BN]; zeros past dk, dv, kv_end
    for (int slot = threadIdx.x; slot < BN * kvecs; slot += 256) {
      const int row = slot / kvecs, v = slot - row * kvecs;
      const int j = t0 + row;
      short8_t x{};
      if (j < kv_end && v * 8 < dk) {
        const int64_t page = table[j / ps];
        x = *reinterpret_cast<const short8_t*>(
            kcache + ((page * G + g) * ps + (j % ps)) * dk + v * 8);
      }
      *reinterpret_cast<short8_t*>(k_lds + row * KS + v * 8) = x;
    }
    // consecutive threads take consecutive keys of one channel group, so
    // the transposed 2-byte LDS writes fall in consecutive banks
    for (int slot = threadIdx.x; slot < BN * vvecs; slot += 256) {
      const int v = slot / BN, row = slot - v * BN;
      const int j = t0 + row;
      short8_t x{};
      if (j < kv_end && v * 8 < dv) {
        const int64_t page = table[j / ps];
        x = *reinterpret_cast<const short8_t*>(
            vcache + ((page * G + g) * ps + (j % ps)) * dv + v * 8);
      }
#pragma unroll
      for (int e = 0; e < 8; e++) vt_lds[(v * 8 + e) * VS + row] = x[e];
    }
    __syncthreads();

    // ---- S = Q K^T: block n covers keys t0 + 16 n + lr
    f32x4_t s[4];
#pragma unroll
    for (int n = 0; n < 4; n++) {
      f32x4_t a{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kc = 0; kc < KC; kc++) {
        const short8_t kb = *reinterpret_cast<const short8_t*>(
            k_lds + (n * 16 + lr) * KS + kc * 32 + lg * 8);
        short8_t tmp = kb;
        a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            q_frag[kc], *reinterpret_cast<bf16x8_t*>(&tmp), a, 0, 0, 0);
      }
      s[n] = a;
    }
    // ---- fp32: scale, penalty, mask, online softmax (rows 4 lg + r)
    float p[4][4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
      float mt = -INFINITY;
#pragma unroll
      for (int n = 0; n < 4; n++) {
        const int j = t0 + n * 16 + lr;
        float x = s[n][r] * qmul[r];
        if (has_bias) x -= b1 * log1pf(b2 * (float)max(pos_r[r] - j, 0));
        x = j <= pos_r[r] ? x : -INFINITY;
        p[n][r] = x;
        mt = fmaxf(mt, x);
      }
      mt = fmaxf(mt, __shfl_xor(mt, 1, 64));
      mt = fmaxf(mt, __shfl_xor(mt, 2, 64));
      mt = fmaxf(mt, __shfl_xor(mt, 4, 64));
      mt = fmaxf(mt, __shfl_xor(mt, 8, 64));
      const float mn = fmaxf(m[r], mt);  // finite from the first block on
      const float corr = expf(m[r] - mn);
      float rs = 0.f;
#pragma unroll
      for (int n = 0; n < 4; n++) {
        p[n][r] = expf(p[n][r] - mn);
        rs += p[n][r];
      }
      rs += __shfl_xor(rs, 1, 64);
      rs += __shfl_xor(rs, 2, 64);
      rs += __shfl_xor(rs, 4, 64);
      rs += __shfl_xor(rs, 8, 64);
      l[r] = l[r] * corr + rs;
      m[r] = mn;
#pragma unroll
      for (int d = 0; d < DN; d++) acc_o[d][r] *= corr;
    }
    // ---- weights to LDS in the A layout of the second product, as a
    // bf16 pair hi + lo (about 16 bits of mantissa, so the product below
    // sees the fp32 weights almost exactly). lo reuses the K block, which
    // every wave has finished reading once the barrier is passed.
    __syncthreads();
    short* pw = p_lds + wid * 16 * VS;
    short* pl = k_lds + wid * 16 * VS;
#pragma unroll
    for (int r = 0; r < 4; r++)
#pragma unroll
      for (int n = 0; n < 4; n++) {
        const bf16_t hi = from_f<bf16_t>(p[n][r]);
        const bf16_t lo = from_f<bf16_t>(p[n][r] - to_f(hi));
        pw[(lg * 4 + r) * VS + n * 16 + lr] = (short)hi;
        pl[(lg * 4 + r) * VS + n * 16 + lr] = (short)lo;
      }
    __syncthreads();
    // ---- O += P V
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
      short8_t pa = *reinterpret_cast<const short8_t*>(
          pw + lr * VS + kt * 32 + lg * 8);
      short8_t pb = *reinterpret_cast<const short8_t*>(
          pl + lr * VS + kt * 32 + lg * 8);
#pragma unroll
      for (int d = 0; d < DN; d++) {
        short8_t vb = *reinterpret_cast<const short8_t*>(
            vt_lds + (d * 16 + lr) * VS + kt * 32 + lg * 8);
        acc_o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            *reinterpret_cast<bf16x8_t*>(&pa),
            *reinterpret_cast<bf16x8_t*>(&vb), acc_o[d], 0, 0, 0);
        acc_o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            *reinterpret_cast<bf16x8_t*>(&pb),
            *reinterpret_cast<bf16x8_t*>(&vb), acc_o[d], 0, 0, 0);
      }
    }
  }
  // ---- normalise and store rows 4 lg + r, channels 16 d + lr
#pragma unroll
  for (int r = 0; r < 4; r++) {
    if (!ok_r[r]) continue;
    const float inv = 1.f / l[r];
    bf16_t* o = out + ((int64_t)(row0 + wid * 16 + lg * 4 + r) * H + h) * dv;
#pragma unroll
    for (int d = 0; d < DN; d++) {
      const int ch = d * 16 + lr;
      if (ch < dv) o[ch] = from_f<bf16_t>(acc_o[d][r] * inv);
    }
  }
}

template <int KC, int DN>
void launch(dim3 grid, size_t lds, bf16_t* out, const bf16_t* proj,
            int proj_stride, int off_q, const bf16_t* kc, const bf16_t* vc,
            const int* pt, int pts, const int* tr0, const int* trn,
            const int* tok_seq, const int* positions, const float* r1,
            const float* r2, int H, int G, int dk, int dv, int ps, float scale,
            float temp_coef, int temp_every, int has_bias) {
  hipLaunchKernelGGL((biased_attention_mfma_kernel<KC, DN>), grid, dim3(256),
                     lds, cur_stream(), out, proj, proj_stride, off_q, kc, vc,
                     pt, pts, tr0, trn, tok_seq, positions, r1, r2, H, G, dk,
                     dv, ps, scale, temp_coef, temp_every, has_bias);
}

inline size_t lds_bytes(int KC, int DN) {
  return (size_t)(BN * (KC * 32 + PADE) + DN * 16 * (BN + PADE) +
                  4 * 16 * (BN + PADE)) * sizeof(short);
}

}  // namespace

// Whether the matrix-core kernel covers these sizes (bf16 caches only).
bool biased_attention_mfma_supported(int64_t dk, int64_t dv) {
  if (dk % 8 || dv % 8 || dk > 256 || dv > 256) return false;
  const int KC = dk <= 64 ? 2 : (dk <= 128 ? 4 : 8);
  const int DN = dv <= 64 ? 4 : (dv <= 128 ? 8 : 16);
  return lds_bytes(KC, DN) <= 64 * 1024;
}

// Rows are given as tiles: tile i covers rows [tile_row0[i], + tile_rows[i])
// (at most 64, consecutive positions of one sequence).
void biased_attention_mfma(torch::Tensor out, torch::Tensor proj, int64_t off_q,
                           torch::Tensor kcache, torch::Tensor vcache,
                           torch::Tensor page_table, torch::Tensor tile_row0,
                           torch::Tensor tile_rows, int64_t max_tile_rows,
                           torch::Tensor tok_seq, torch::Tensor positions,
                           c10::optional<torch::Tensor> r1,
                           c10::optional<torch::Tensor> r2, double scale,
                           double temp_coef, int64_t temp_every) {
  const int T_ = out.size(0), H = out.size(1), dv = out.size(2);
  const int G = kcache.size(1), ps = kcache.size(2), dk = kcache.size(3);
  const int NT = tile_row0.size(0);
  SEQ_CHECK(out.scalar_type() == torch::kBFloat16 && out.is_contiguous() &&
                proj.scalar_type() == torch::kBFloat16 &&
                kcache.scalar_type() == torch::kBFloat16 &&
                vcache.scalar_type() == torch::kBFloat16, "mfma attention is bf16");
  SEQ_CHECK(kcache.is_contiguous() && vcache.is_contiguous() &&
                vcache.size(3) == dv && vcache.size(1) == G &&
                vcache.size(2) == ps && H % G == 0, "mfma attention cache");
  SEQ_CHECK(biased_attention_mfma_supported(dk, dv), "mfma attention sizes");
  SEQ_CHECK(reinterpret_cast<uintptr_t>(kcache.data_ptr()) % 16 == 0 &&
                reinterpret_cast<uintptr_t>(vcache.data_ptr()) % 16 == 0,
            "mfma attention cache alignment");
  SEQ_CHECK(proj.stride(1) == 1 && proj.size(0) == T_ &&
                off_q + H * dk <= proj.size(1), "mfma attention q");
  SEQ_CHECK(page_table.scalar_type() == torch::kInt && page_table.dim() == 2 &&
                page_table.stride(1) == 1, "page table");
  for (const torch::Tensor* t : {&tok_seq, &positions})
    SEQ_CHECK(t->scalar_type() == torch::kInt && t->is_contiguous() &&
                  t->numel() >= T_, "token descriptors");
  for (const torch::Tensor* t : {&tile_row0, &tile_rows})
    SEQ_CHECK(t->scalar_type() == torch::kInt && t->is_contiguous() &&
                  t->numel() == NT && t->is_cuda(), "tile descriptors");
  SEQ_CHECK(max_tile_rows >= 1 && max_tile_rows <= 64, "tile height");
  SEQ_CHECK(r1.has_value() == r2.has_value(), "bias parameters");
  if (r1)
    SEQ_CHECK(r1->scalar_type() == torch::kFloat && r1->numel() == H &&
                  r2->scalar_type() == torch::kFloat && r2->numel() == H,
              "bias parameters");
  SEQ_CHECK(temp_every >= 1, "temperature period");
  if (NT == 0) return;
  const int KC = dk <= 64 ? 2 : (dk <= 128 ? 4 : 8);
  const int DN = dv <= 64 ? 4 : (dv <= 128 ? 8 : 16);
  const size_t lds = lds_bytes(KC, DN);
#define ARGS                                                                  \
  dim3(NT, H), lds, ptr<bf16_t>(out), cptr<bf16_t>(proj),                     \
      (int)proj.stride(0), (int)off_q, cptr<bf16_t>(kcache),                  \
      cptr<bf16_t>(vcache), cptr<int>(page_table), (int)page_table.stride(0), \
      cptr<int>(tile_row0), cptr<int>(tile_rows), cptr<int>(tok_seq),         \
      cptr<int>(positions), r1 ? cptr<float>(*r1) : nullptr,                  \
      r2 ? cptr<float>(*r2) : nullptr, H, G, dk, dv, ps, (float)scale,        \
      (float)temp_coef, (int)temp_every, r1 ? 1 : 0
  if (KC == 2 && DN == 4) launch<2, 4>(ARGS);
  else if (KC == 2 && DN == 8) launch<2, 8>(ARGS);
  else if (KC == 2 && DN == 16) launch<2, 16>(ARGS);
  else if (KC == 4 && DN == 4) launch<4, 4>(ARGS);
  else if (KC == 4 && DN == 8) launch<4, 8>(ARGS);
  else if (KC == 4 && DN == 16) launch<4, 16>(ARGS);
  else if (KC == 8 && DN == 4) launch<8, 4>(ARGS);
  else if (KC == 8 && DN == 8) launch<8, 8>(ARGS);
  else TORCH_CHECK(false, "seqmix: mfma attention sizes");
#undef ARGS
}
