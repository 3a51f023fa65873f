// Between the q/k/v projection and attention, for mixers whose keys and values differ in width or whose queries and
// keys are normed as whole rows: one kernel per step and layer that norms, turns, blends and writes the cache.
// All arithmetic is float32 (angles in float64 where the caller gives the table's float64 remainder); only loads and
// stores see the storage type.
#include "common.h"
#include "sprout_hip.h"

namespace sprout {

struct PrepareArgs {
  const void* proj;            // [T, stride]: q (nq * dim), k (nkv * dim), v (nkv * vdim) of a token, biases already added
  long long stride;
  int nq, nkv, dim, vdim, width;   // width: numbers a head takes in q_out and in the pools (>= dim, vdim; zeros behind)
  const void* q_norm;          // [nq * dim], [nkv * dim]: RMS norm over the whole q row and the whole k row (null: none)
  const void* k_norm;
  float eps;
  const int32_t* positions;
  const float* inv_freq;       // [rotary_dim / 2]; rotary_dim == 0: nothing turns
  const float* inv_freq_tail;  // the float64 table minus inv_freq (null: angles in float32)
  int rotary_dim;
  const void* blend;           // one number lambda: v <- (1 - lambda) v + lambda first (null: v as projected)
  void* first;                 // [T, nkv * vdim]: written with v where keep_first, read where blend is given
  int keep_first;
  const int32_t* slot_mapping; // null: nothing is cached
  void* k_pool;                // [pages][nkv][page_size][width]
  void* v_pool;                // [pages][nkv][width][page_size]
  int page_size;
  void* q_out;                 // [T, nq * width]
};

// One block a token.
template <typename T>
__global__ __launch_bounds__(256) void qkv_prepare_kernel(PrepareArgs a) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const T* row = (const T*)a.proj + size_t(t) * a.stride;
  const int nq = a.nq, nkv = a.nkv, D = a.dim, V = a.vdim, W = a.width;
  const T* qrow = row;
  const T* krow = row + size_t(nq) * D;
  const T* vrow = krow + size_t(nkv) * D;
  float q_scale = 1.f, k_scale = 1.f;
  if (a.q_norm) {
    float sq = 0.f;
    for (int i = threadIdx.x; i < nq * D; i += blockDim.x) { const float x = to_float(qrow[i]); sq = fmaf(x, x, sq); }
    q_scale = 1.0f / sqrtf(block_sum(sq, scratch) / float(nq * D) + a.eps);
    sq = 0.f;
    for (int i = threadIdx.x; i < nkv * D; i += blockDim.x) { const float x = to_float(krow[i]); sq = fmaf(x, x, sq); }
    k_scale = 1.0f / sqrtf(block_sum(sq, scratch) / float(nkv * D) + a.eps);
  }
  const int slot = a.slot_mapping ? a.slot_mapping[t] : -1;
  const int page = slot >= 0 ? slot / a.page_size : 0, off = slot >= 0 ? slot % a.page_size : 0;
  const int half = a.rotary_dim / 2;
  const int pos = a.positions ? a.positions[t] : 0;

  // queries and keys: head by head, number by number of the padded head; a thread that owns the first of a turning
  // pair also writes its partner
  const int heads = nq + nkv;
  for (int i = threadIdx.x; i < heads * W; i += blockDim.x) {
    const int head = i / W, d = i % W;
    const bool is_q = head < nq;
    T* dst = nullptr;
    if (is_q) dst = (T*)a.q_out + (size_t(t) * nq + head) * W;
    else if (slot >= 0) dst = (T*)a.k_pool + ((size_t(page) * nkv + (head - nq)) * a.page_size + off) * W;
    if (!dst) continue;
    if (d >= D) { dst[d] = from_float<T>(0.f); continue; }
    if (d >= half && d < 2 * half) continue;          // written by the owner of its pair
    const T* src = is_q ? qrow + size_t(head) * D : krow + size_t(head - nq) * D;
    const T* nw = is_q ? (const T*)a.q_norm : (const T*)a.k_norm;
    const float scale = is_q ? q_scale : k_scale;
    const int col = (is_q ? head : head - nq) * D;
    auto normed = [&](int e) {
      float x = to_float(src[e]);
      if (nw) x = to_float(from_float<T>((x * scale) * to_float(nw[col + e])));   // the storage type's rounding, as a norm kernel would leave it
      return x;
    };
    if (d >= 2 * half) { dst[d] = from_float<T>(normed(d)); continue; }
    float sn, cs;
    if (a.inv_freq_tail) {
      double sn64, cs64;
      sincos(double(pos) * (double(a.inv_freq[d]) + double(a.inv_freq_tail[d])), &sn64, &cs64);
      sn = float(sn64);
      cs = float(cs64);
    } else {
      sincosf(float(pos) * a.inv_freq[d], &sn, &cs);
    }
    const float x = normed(d), y = normed(d + half);
    dst[d] = from_float<T>(x * cs - y * sn);
    dst[d + half] = from_float<T>(y * cs + x * sn);
  }

  // values: blended with the first flagged layer's, kept for the later layers, written dimension-major
  const float lam = a.blend ? to_float(*(const T*)a.blend) : 0.f;
  T* first = a.first ? (T*)a.first + size_t(t) * nkv * V : nullptr;
  for (int i = threadIdx.x; i < nkv * W; i += blockDim.x) {
    const int g = i / W, d = i % W;
    float v = 0.f;
    if (d < V) {
      v = to_float(vrow[g * V + d]);
      if (a.blend) v = to_float(from_float<T>((1.0f - lam) * v + lam * to_float(first[g * V + d])));
      else if (a.keep_first) first[g * V + d] = from_float<T>(v);
    }
    if (slot >= 0) ((T*)a.v_pool)[((size_t(page) * nkv + g) * W + d) * a.page_size + off] = from_float<T>(v);
  }
}

}  // namespace sprout

using namespace sprout;

extern "C" int sp_qkv_prepare(void* stream, int dtype, const void* proj, long long stride, int nq, int nkv, int dim, int vdim,
                              int width, const void* q_norm, const void* k_norm, float eps, const int32_t* positions,
                              const float* inv_freq, const float* inv_freq_tail, int rotary_dim, const void* blend,
                              void* first, int keep_first, const int32_t* slot_mapping, void* k_pool, void* v_pool,
                              int page_size, int num_pages, void* q_out, int T) {
  SP_REQUIRE(T >= 0 && nq > 0 && nkv > 0 && dim > 0 && vdim > 0 && width >= dim && width >= vdim,
             "sp_qkv_prepare: bad sizes nq=%d nkv=%d dim=%d vdim=%d width=%d", nq, nkv, dim, vdim, width);
  SP_REQUIRE(stride >= (long long)(nq + nkv) * dim + (long long)nkv * vdim, "sp_qkv_prepare: a row of %lld numbers does not hold q, k and v", stride);
  SP_REQUIRE(proj && q_out, "sp_qkv_prepare: null operand");
  SP_REQUIRE((q_norm == nullptr) == (k_norm == nullptr), "sp_qkv_prepare: queries and keys are normed together or not at all");
  SP_REQUIRE(rotary_dim >= 0 && rotary_dim % 2 == 0 && rotary_dim <= dim, "sp_qkv_prepare: %d numbers cannot turn in a head of %d", rotary_dim, dim);
  SP_REQUIRE(rotary_dim == 0 || (positions && inv_freq), "sp_qkv_prepare: a rotation needs positions and frequencies");
  SP_REQUIRE(!(blend || keep_first) || first, "sp_qkv_prepare: blending values needs the buffer of the first layer's");
  SP_REQUIRE(!slot_mapping || (k_pool && v_pool && page_size > 0 && num_pages > 0), "sp_qkv_prepare: bad cache geometry");
  if (T == 0) return 0;
  PrepareArgs a = {proj, stride, nq, nkv, dim, vdim, width, q_norm, k_norm, eps, positions, inv_freq, inv_freq_tail, rotary_dim,
                   blend, first, keep_first, slot_mapping, k_pool, v_pool, page_size, q_out};
  hipStream_t s = (hipStream_t)stream;
  if (dtype == kF32) qkv_prepare_kernel<float><<<T, 256, 0, s>>>(a);
  else if (dtype == kBF16) qkv_prepare_kernel<bf16_t><<<T, 256, 0, s>>>(a);
  else SP_REQUIRE(false, "sp_qkv_prepare: unsupported dtype %d", dtype);
  return check_launch("sp_qkv_prepare");
}
