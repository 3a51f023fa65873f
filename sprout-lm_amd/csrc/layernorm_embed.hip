// Layer norm (bias optional), and the token embedding with a hashed-pair (bigram) table added.
// All arithmetic is float32; only loads and stores see the storage type.
#include "common.h"
#include "sprout_hip.h"

namespace sprout {

// y = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w (+ b where b is given).  One block a row; the row is read three times (the second
// and third time from the caches): the variance is the mean of the squared deviations, not E[x^2] - mean^2.
// With w2 and out2 the same normalised row is also written times a second weight (two norms of one input).
template <typename TW, typename TO>
__global__ void layernorm_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows,
                                 const TW* __restrict__ w, const TW* __restrict__ w2, const TW* __restrict__ b,
                                 const TW* __restrict__ b2, float eps, TO* __restrict__ out, TO* __restrict__ out2, int H) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const float* in = x + size_t(rows ? rows[r] : r) * H;
  TO* o = out + size_t(r) * H;
  TO* o2 = out2 ? out2 + size_t(r) * H : nullptr;
  constexpr int KEEP = 8;
  if (H <= KEEP * int(blockDim.x)) {      // the row stays in registers: one trip to memory
    float v[KEEP];
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < KEEP; ++j) {
      const int i = threadIdx.x + j * blockDim.x;
      v[j] = i < H ? in[i] : 0.f;
      sum += v[j];
    }
    const float mean = block_sum(sum, scratch) / float(H);
    float sq = 0.f;
#pragma unroll
    for (int j = 0; j < KEEP; ++j) {
      const float d = threadIdx.x + j * blockDim.x < H ? v[j] - mean : 0.f;
      sq = fmaf(d, d, sq);
    }
    const float scale = 1.0f / sqrtf(block_sum(sq, scratch) / float(H) + eps);
#pragma unroll
    for (int j = 0; j < KEEP; ++j) {
      const int i = threadIdx.x + j * blockDim.x;
      if (i >= H) continue;
      const float y = (v[j] - mean) * scale;
      o[i] = from_float<TO>(fmaf(y, to_float(w[i]), b ? to_float(b[i]) : 0.f));
      if (o2) o2[i] = from_float<TO>(fmaf(y, to_float(w2[i]), b2 ? to_float(b2[i]) : 0.f));
    }
    return;
  }
  float sum = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) sum += in[i];
  const float mean = block_sum(sum, scratch) / float(H);
  float sq = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float d = in[i] - mean;
    sq = fmaf(d, d, sq);
  }
  const float scale = 1.0f / sqrtf(block_sum(sq, scratch) / float(H) + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float y = (in[i] - mean) * scale;
    o[i] = from_float<TO>(fmaf(y, to_float(w[i]), b ? to_float(b[i]) : 0.f));
    if (o2) o2[i] = from_float<TO>(fmaf(y, to_float(w2[i]), b2 ? to_float(b2[i]) : 0.f));
  }
}

// residual[t] = table[token] + pairs[row], row = (previous * mul_prev + token * mul_cur) mod buckets, and row
// `buckets` for a sequence's first token (position 0).  The previous token of a step's first token of a sequence
// is what `last_token[state_slots[seq]]` holds from the step before; the block of that first token then leaves
// the step's last token of the sequence there (nobody else reads or writes that entry in this launch).
template <typename TW>
__global__ void embed_bigram_kernel(const TW* __restrict__ table, const TW* __restrict__ pairs,
                                    const int32_t* __restrict__ tokens, const int32_t* __restrict__ positions,
                                    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
                                    const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ state_slots,
                                    int32_t* __restrict__ last_token, float* __restrict__ residual, int H,
                                    long long buckets, long long mul_prev, long long mul_cur) {
  __shared__ long long row_s;
  const int t = blockIdx.x;
  const int cur = tokens[t];
  if (threadIdx.x == 0) {
    const int s = seq_of_token[t];
    const int first = q_start[s];
    long long row = buckets;
    int previous = 0;
    if (t == first) {
      int32_t* kept = last_token + state_slots[s];
      previous = *kept;
      *kept = tokens[first + q_len[s] - 1];
    } else {
      previous = tokens[t - 1];
    }
    // (a * m) mod b = (a * (m mod b)) mod b: with the multipliers reduced first the products stay far inside 64 bits
    if (positions[t] > 0) row = (((long long)previous * (mul_prev % buckets)) % buckets + ((long long)cur * (mul_cur % buckets)) % buckets) % buckets;
    row_s = row;
  }
  __syncthreads();
  const TW* a = table + size_t(cur) * H;
  const TW* b = pairs + size_t(row_s) * H;
  float* out = residual + size_t(t) * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = to_float(a[i]) + to_float(b[i]);
}

}  // namespace sprout

using namespace sprout;

extern "C" int sp_layernorm(void* stream, const float* x, const int32_t* rows, int w_dtype, const void* w, const void* w2,
                            const void* b, const void* b2, float eps, int out_dtype, void* out, void* out2, int R, int H) {
  SP_REQUIRE(R >= 0 && H > 0 && x && w && out, "sp_layernorm: bad arguments R=%d H=%d", R, H);
  SP_REQUIRE((w2 == nullptr) == (out2 == nullptr), "sp_layernorm: a second weight goes with a second output");
  SP_REQUIRE(!b2 || w2, "sp_layernorm: a second bias goes with a second weight");
  if (R == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int threads = H >= 2048 ? 512 : 256;
#define SP_LN(TW, TO) \
  layernorm_kernel<TW, TO><<<R, threads, 0, s>>>(x, rows, (const TW*)w, (const TW*)w2, (const TW*)b, (const TW*)b2, eps, \
                                                (TO*)out, (TO*)out2, H)
  if (w_dtype == kF32 && out_dtype == kF32) SP_LN(float, float);
  else if (w_dtype == kF32 && out_dtype == kBF16) SP_LN(float, bf16_t);
  else if (w_dtype == kBF16 && out_dtype == kF32) SP_LN(bf16_t, float);
  else if (w_dtype == kBF16 && out_dtype == kBF16) SP_LN(bf16_t, bf16_t);
  else SP_REQUIRE(false, "sp_layernorm: unsupported dtypes w=%d out=%d", w_dtype, out_dtype);
#undef SP_LN
  return check_launch("sp_layernorm");
}

extern "C" int sp_embed_bigram(void* stream, int table_dtype, const void* table, const void* pairs,
                               const int32_t* tokens, const int32_t* positions, const int32_t* q_start,
                               const int32_t* q_len, const int32_t* seq_of_token, const int32_t* state_slots,
                               int32_t* last_token, float* residual, int T, int H, int V, long long buckets,
                               long long mul_prev, long long mul_cur) {
  SP_REQUIRE(T >= 0 && H > 0 && V > 0 && buckets > 0 && mul_prev >= 0 && mul_cur >= 0,
             "sp_embed_bigram: bad sizes T=%d H=%d V=%d buckets=%lld", T, H, V, buckets);
  SP_REQUIRE(table && pairs && tokens && positions && q_start && q_len && seq_of_token && state_slots && last_token &&
                 residual, "sp_embed_bigram: null operand");
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (table_dtype == kF32)
    embed_bigram_kernel<float><<<T, 256, 0, s>>>((const float*)table, (const float*)pairs, tokens, positions, q_start,
                                                 q_len, seq_of_token, state_slots, last_token, residual, H, buckets,
                                                 mul_prev, mul_cur);
  else if (table_dtype == kBF16)
    embed_bigram_kernel<bf16_t><<<T, 256, 0, s>>>((const bf16_t*)table, (const bf16_t*)pairs, tokens, positions,
                                                  q_start, q_len, seq_of_token, state_slots, last_token, residual, H,
                                                  buckets, mul_prev, mul_cur);
  else
    SP_REQUIRE(false, "sp_embed_bigram: unsupported table dtype %d", table_dtype);
  return check_launch("sp_embed_bigram");
}
