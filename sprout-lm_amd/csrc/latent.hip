// Attention over a latent: what stands between the input projections and the attention kernel.
//
// A token's projections lie in one row `proj`: per head [dim unrotated, rot rotated] query numbers from column
// q_off on, then at dkv_off the latent (rank numbers, RMS-normed here) and one rotated key part (rot numbers)
// shared by all heads.  The cache holds per token the key [latent, rotated part] (rank + rot numbers, one
// key/value head) and as value the latent in the same width (the rotated part's columns of the value pool are never
// written and stay zero), so that every attention kernel for one key/value head and heads of rank + rot takes it.
// Queries for that attention are [query . U_k (rank numbers, written by the per-head product), rotated part]:
// this kernel writes the rotated part.
//
// Rotation: the first rot_dims numbers of a rotated part turn, (2i, 2i + 1) together, by position * freq[i], and
// cosine and sine are multiplied by `magnitude`; the rest pass unchanged.  exact != 0: angle, sine and cosine in
// float64 (the float32 path), else float32.
#include "common.h"
#include "sprout_hip.h"

namespace sprout {

template <typename T, typename TW>
__global__ void latent_prepare_kernel(const T* __restrict__ proj, int proj_stride, int q_off, int heads, int dim, int rot,
                                      int dkv_off, int rank, const TW* __restrict__ norm_w, float eps,
                                      const int32_t* __restrict__ positions, const double* __restrict__ freq,
                                      int rot_dims, float magnitude, int exact, const int32_t* __restrict__ slot_mapping,
                                      T* __restrict__ k_pool, T* __restrict__ v_pool, int page_size,
                                      T* __restrict__ q_out) {
  extern __shared__ float cs[];      // [rot_dims / 2][2] cosine, sine (times magnitude)
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const T* row = proj + size_t(t) * proj_stride;
  const int pos = positions[t];
  for (int i = threadIdx.x; i < rot_dims / 2; i += blockDim.x) {
    float c, s;
    if (exact) {
      const double a = double(pos) * freq[i];
      c = float(cos(a) * double(magnitude));
      s = float(sin(a) * double(magnitude));
    } else {
      const float a = float(pos) * float(freq[i]);
      c = cosf(a) * magnitude;
      s = sinf(a) * magnitude;
    }
    cs[2 * i] = c;
    cs[2 * i + 1] = s;
  }
  float sum = 0.f;
  for (int d = threadIdx.x; d < rank; d += blockDim.x) {
    const float v = to_float(row[dkv_off + d]);
    sum = fmaf(v, v, sum);
  }
  sum = block_sum(sum, scratch);      // (its barriers also publish cs)
  const float scale = 1.0f / sqrtf(sum / float(rank) + eps);
  const int width = rank + rot;
  const int slot = slot_mapping ? slot_mapping[t] : -1;

  auto turned = [&](const T* part, int d) -> float {
    if (d >= rot_dims) return to_float(part[d]);
    const int i = d >> 1;
    const float u = to_float(part[2 * i]), v = to_float(part[2 * i + 1]);
    const float c = cs[2 * i], s = cs[2 * i + 1];
    return (d & 1) ? v * c + u * s : u * c - v * s;
  };

  if (slot >= 0) {
    const int page = slot / page_size, off = slot - page * page_size;
    T* key = k_pool + (size_t(page) * page_size + off) * width;
    T* value = v_pool + size_t(page) * width * page_size + off;      // [page][dim][token]
    for (int d = threadIdx.x; d < rank; d += blockDim.x) {
      const T c = from_float<T>((to_float(row[dkv_off + d]) * scale) * to_float(norm_w[d]));
      key[d] = c;
      value[size_t(d) * page_size] = c;
    }
    for (int d = threadIdx.x; d < rot; d += blockDim.x) key[rank + d] = from_float<T>(turned(row + dkv_off + rank, d));
  }
  for (int j = threadIdx.x; j < heads * rot; j += blockDim.x) {
    const int h = j / rot, d = j - h * rot;
    q_out[(size_t(t) * heads + h) * width + rank + d] = from_float<T>(turned(row + q_off + h * (dim + rot) + dim, d));
  }
}

}  // namespace sprout

using namespace sprout;

extern "C" int sp_latent_prepare(void* stream, int dtype, const void* proj, int proj_stride, int q_off, int heads, int dim,
                                 int rot, int dkv_off, int rank, int norm_w_dtype, const void* norm_w, float eps,
                                 const int32_t* positions, const double* freq, int rot_dims, float magnitude, int exact,
                                 const int32_t* slot_mapping, void* k_pool, void* v_pool, int page_size, int num_pages,
                                 void* q_out, int T) {
  SP_REQUIRE(T >= 0 && heads > 0 && dim >= 0 && rot >= 0 && rank > 0, "sp_latent_prepare: bad sizes");
  SP_REQUIRE(rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0, "sp_latent_prepare: %d of %d numbers turn", rot_dims, rot);
  SP_REQUIRE(q_off >= 0 && dkv_off >= 0 && proj_stride >= q_off + heads * (dim + rot) && proj_stride >= dkv_off + rank + rot,
             "sp_latent_prepare: a row of %d numbers does not hold the projections", proj_stride);
  SP_REQUIRE(proj && norm_w && positions && q_out && (rot_dims == 0 || freq), "sp_latent_prepare: null operand");
  SP_REQUIRE(!slot_mapping || (k_pool && v_pool && page_size > 0 && num_pages > 0), "sp_latent_prepare: no pools to write to");
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = size_t(rot_dims > 0 ? rot_dims : 2) * sizeof(float);
#define SP_LATENT(TT, TW)                                                                                            \
  latent_prepare_kernel<TT, TW><<<T, 256, lds, s>>>((const TT*)proj, proj_stride, q_off, heads, dim, rot, dkv_off, rank, \
                                                    (const TW*)norm_w, eps, positions, freq, rot_dims, magnitude, exact, \
                                                    slot_mapping, (TT*)k_pool, (TT*)v_pool, page_size, (TT*)q_out)
  if (dtype == kF32 && norm_w_dtype == kF32) SP_LATENT(float, float);
  else if (dtype == kBF16 && norm_w_dtype == kBF16) SP_LATENT(bf16_t, bf16_t);
  else if (dtype == kBF16 && norm_w_dtype == kF32) SP_LATENT(bf16_t, float);
  else if (dtype == kF32 && norm_w_dtype == kBF16) SP_LATENT(float, bf16_t);
  else SP_REQUIRE(false, "sp_latent_prepare: unsupported dtypes %d, %d", dtype, norm_w_dtype);
#undef SP_LATENT
  return check_launch("sp_latent_prepare");
}
