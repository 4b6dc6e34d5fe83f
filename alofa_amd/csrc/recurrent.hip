// Kernels of layers that carry state of fixed size per request instead of (or beside) pages of keys:
// a short causal convolution over time, the mix of a token with the one before it, and the linear
// recurrence S_t = diag(w_t) S_(t-1) + k_t v_t^T with its read-out, which serves retention (one decay per
// head), gated linear attention (a decay per key channel and token) and RWKV-style time mixing (the same with
// the read-out taken before the update and a bonus for the current token).
//
// How a step's rows belong to requests: request r of the step owns the rows row_off[r] .. row_off[r+1]-1,
// in position order, and keeps its state in slot req_slot[r]. With row_off absent every request brings one
// row (row r). req_of_row[t] names the request of row t (absent: t itself). What came before a request's
// first row of this step is in its state, which is zero for a new request, so no kernel asks for positions.
//
// State and all arithmetic of the recurrences are float; q, k, v and gates come in the activation type.
#include "common.h"

namespace alofa {

// ---- short causal convolution ------------------------------------------------------------------------
// out[t, c] = h[t, c] + sum_j w[c, j] * h[t - taps + 1 + j, c], rows before the request's first row of this step
// taken from state[slot, i, c], which holds the last taps - 1 inputs (i = taps - 2 is the newest). The state
// is not written here: rows of one request are spread over blocks that all read it.
template <typename TO, typename TI, typename Acc>
__global__ void __launch_bounds__(256) short_conv_kernel(TO* __restrict__ out, const TI* __restrict__ h, const float* __restrict__ w,
                                                         const TI* __restrict__ state, const int32_t* __restrict__ req_slot,
                                                         const int32_t* __restrict__ row_off, const int32_t* __restrict__ req_of_row,
                                                         int rows, int width, int taps) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<int64_t>(rows) * width) return;
  const int t = static_cast<int>(idx / width), c = static_cast<int>(idx % width);
  const int r = req_of_row ? req_of_row[t] : t;
  const int row0 = row_off ? row_off[r] : r;
  const TI* st = state + static_cast<int64_t>(req_slot[r]) * (taps - 1) * width;
  const float* wc = w + static_cast<int64_t>(c) * taps;
  const Acc mine = static_cast<Acc>(load_f32(h + static_cast<int64_t>(t) * width + c));
  Acc acc = mine;
  for (int j = 0; j < taps; ++j) {
    const int s = t - taps + 1 + j;
    const Acc v = j == taps - 1 ? mine
                  : s >= row0  ? static_cast<Acc>(load_f32(h + static_cast<int64_t>(s) * width + c))
                               : static_cast<Acc>(load_f32(st + static_cast<int64_t>(taps - 1 + s - row0) * width + c));
    acc += static_cast<Acc>(wc[j]) * v;
  }
  store_f32(out + static_cast<int64_t>(t) * width + c, static_cast<float>(acc));
}

// The last `keep` rows a request has seen, after this step: state[slot, i, c] = the input at (end of the request's
// rows) - keep + i, from this step's rows or, where the step brought fewer, from the old state. A thread owns one
// channel of one request, reads what it needs and writes afterwards.
constexpr int kMaxKeep = 8;
template <typename TI>
__global__ void __launch_bounds__(256) keep_last_rows_kernel(TI* __restrict__ state, const TI* __restrict__ h, const int32_t* __restrict__ req_slot,
                                                             const int32_t* __restrict__ row_off, int requests, int width, int keep) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<int64_t>(requests) * width) return;
  const int r = static_cast<int>(idx / width), c = static_cast<int>(idx % width);
  const int row0 = row_off ? row_off[r] : r, end = row_off ? row_off[r + 1] : r + 1;
  TI* st = state + static_cast<int64_t>(req_slot[r]) * keep * width;
  TI kept[kMaxKeep];
#pragma unroll
  for (int i = 0; i < kMaxKeep; ++i) {
    if (i < keep) {
      const int s = end - keep + i;
      kept[i] = s >= row0 ? h[static_cast<int64_t>(s) * width + c] : st[static_cast<int64_t>(keep + s - row0) * width + c];
    }
  }
#pragma unroll
  for (int i = 0; i < kMaxKeep; ++i)
    if (i < keep) st[static_cast<int64_t>(i) * width + c] = kept[i];
}

// ---- mix with the token before --------------------------------------------------------------------------
// out[s, t, c] = x[t, c] + (x[t-1, c] - x[t, c]) * mu[s, c] for s < n_mixes; the row before a request's first row
// of this step is state[slot, c] (zeros for a new request). The state is kept by keep_last_rows (keep = 1).
template <typename T>
__global__ void __launch_bounds__(256) shift_mix_kernel(T* __restrict__ out, const T* __restrict__ x, const float* __restrict__ mu,
                                                        const T* __restrict__ state, const int32_t* __restrict__ req_slot,
                                                        const int32_t* __restrict__ row_off, const int32_t* __restrict__ req_of_row,
                                                        int rows, int width, int n_mixes) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<int64_t>(rows) * width) return;
  const int t = static_cast<int>(idx / width), c = static_cast<int>(idx % width);
  const int r = req_of_row ? req_of_row[t] : t;
  const int row0 = row_off ? row_off[r] : r;
  const float cur = load_f32(x + static_cast<int64_t>(t) * width + c);
  const float prev = t > row0 ? load_f32(x + static_cast<int64_t>(t - 1) * width + c)
                              : load_f32(state + static_cast<int64_t>(req_slot[r]) * width + c);
  const float diff = prev - cur;
  for (int s = 0; s < n_mixes; ++s)
    store_f32(out + (static_cast<int64_t>(s) * rows + t) * width + c, cur + diff * mu[static_cast<int64_t>(s) * width + c]);
}

// ---- the linear recurrence ----------------------------------------------------------------------------------
// Per request and head, a state S [dk, dv] (float, in the request's slot) and for its rows in order:
//   after-update form:   S = diag(w_t) S + k_t v_t^T;  o_t = S^T q_t
//   before-update form:  o_t = (S + diag(u) k_t v_t^T)^T q_t;  S = diag(w_t) S + k_t v_t^T     (bonus u per head and key channel)
// with q scaled by q_scale and k by k_scale first. The decay w_t per key channel comes as
//   kDecayPerHead:     a constant per head (decay[head]),
//   kDecaySigmoidRoot: sigmoid(z)^(1/tau), z = decay_in[t, head * dk + i], formed as exp(log_sigmoid(z) / tau),
//   kDecayExpNegExp:   exp(-exp(z)).
//
// A block owns (request, head, a slice of up to 64 value channels). Lanes are value channels; wave g owns the key channels
// g * KPT .. g * KPT + KPT - 1 and keeps its share of S in registers (KPT floats per lane). Rows go through LDS in chunks:
// all threads fetch the chunk's q, k, decays (made once per row and channel, not per lane) and v; then every wave runs the
// chunk's rows in order against LDS alone, leaving its partial read-outs there; after a barrier they are added over the
// waves in wave order and written. Within a wave the sum over its key channels runs in ascending order, so a read-out
// depends on nothing but the rows before it: not on how rows were cut into steps or chunks.
enum DecayKind : int { kDecayPerHead = 0, kDecaySigmoidRoot = 1, kDecayExpNegExp = 2 };

template <typename T, int KPT>
__global__ void __launch_bounds__(KPT == 64 ? 512 : 256) linear_recurrence_kernel(
    float* __restrict__ out, const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k, int64_t k_stride,
    const T* __restrict__ v, int64_t v_stride, const float* __restrict__ decay_in, int64_t decay_stride, const float* __restrict__ decay_head,
    const float* __restrict__ bonus, float* __restrict__ state, const int32_t* __restrict__ req_slot, const int32_t* __restrict__ row_off,
    int heads, int dk, int dv, int decay_kind, float inv_tau, float q_scale, float k_scale, int before_update, int chunk) {
  extern __shared__ float lds[];
  const int n_waves = blockDim.x / kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int r = blockIdx.z, head = blockIdx.y, j0 = blockIdx.x * kWave;
  const int row0 = row_off ? row_off[r] : r, end = row_off ? row_off[r + 1] : r + 1;
  const int j = j0 + lane;
  const bool live = j < dv;
  const int i0 = wave * KPT;
  // LDS: q, k, w as [chunk][dk_pad]; v as [chunk][64]; partial read-outs as [chunk][waves][64]
  const int dk_pad = n_waves * KPT;
  float* lq = lds;
  float* lk = lq + chunk * dk_pad;
  float* lw = lk + chunk * dk_pad;
  float* lv = lw + chunk * dk_pad;
  float* lp = lv + chunk * kWave;

  float* S_g = state + ((static_cast<int64_t>(req_slot[r]) * heads + head) * dk) * dv;
  float S[KPT], u[KPT];
#pragma unroll
  for (int i = 0; i < KPT; ++i) {
    S[i] = (live && i0 + i < dk) ? S_g[static_cast<int64_t>(i0 + i) * dv + j] : 0.f;
    u[i] = (bonus && i0 + i < dk) ? bonus[head * dk + i0 + i] : 0.f;
  }
  const float head_decay = decay_kind == kDecayPerHead ? decay_head[head] : 1.f;

  for (int c0 = row0; c0 < end; c0 += chunk) {
    const int n = min(chunk, end - c0);
    __syncthreads();      // the chunk before is written out; LDS is free again
    for (int e = threadIdx.x; e < n * dk_pad; e += blockDim.x) {
      const int tt = e / dk_pad, i = e % dk_pad;
      const int64_t t = c0 + tt;
      float qv = 0.f, kv = 0.f, wv = 1.f;
      if (i < dk) {
        qv = load_f32(q + t * q_stride + head * dk + i) * q_scale;
        kv = load_f32(k + t * k_stride + head * dk + i) * k_scale;
        if (decay_kind == kDecayPerHead) {
          wv = head_decay;
        } else {
          const float z = decay_in[t * decay_stride + head * dk + i];
          if (decay_kind == kDecaySigmoidRoot) {
            // log sigmoid(z) = -(max(-z, 0) + log1p(exp(-|z|)))
            const float ls = -(fmaxf(-z, 0.f) + log1pf(expf(-fabsf(z))));
            wv = expf(ls * inv_tau);
          } else {
            wv = expf(-expf(z));
          }
        }
      }
      lq[e] = qv;
      lk[e] = kv;
      lw[e] = wv;
    }
    for (int e = threadIdx.x; e < n * kWave; e += blockDim.x) {
      const int tt = e / kWave, jj = e % kWave;
      lv[e] = j0 + jj < dv ? load_f32(v + static_cast<int64_t>(c0 + tt) * v_stride + head * dv + j0 + jj) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const float vj = lv[tt * kWave + lane];
      const float* pq = lq + tt * dk_pad + i0;
      const float* pk = lk + tt * dk_pad + i0;
      const float* pw = lw + tt * dk_pad + i0;
      float acc = 0.f;
      if (before_update) {
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
          const float kvv = pk[i] * vj;
          acc += pq[i] * (S[i] + u[i] * kvv);
          S[i] = pw[i] * S[i] + kvv;
        }
      } else {
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
          S[i] = pw[i] * S[i] + pk[i] * vj;
          acc += pq[i] * S[i];
        }
      }
      lp[(tt * n_waves + wave) * kWave + lane] = acc;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < n * kWave; e += blockDim.x) {
      const int tt = e / kWave, jj = e % kWave;
      if (j0 + jj < dv) {
        float acc = 0.f;
        for (int g = 0; g < n_waves; ++g) acc += lp[(tt * n_waves + g) * kWave + jj];
        out[(static_cast<int64_t>(c0 + tt) * heads + head) * dv + j0 + jj] = acc;
      }
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < KPT; ++i)
      if (i0 + i < dk) S_g[static_cast<int64_t>(i0 + i) * dv + j] = S[i];
  }
}

}  // namespace alofa

using namespace alofa;

static inline unsigned blocks_of(int64_t n) { return static_cast<unsigned>((n + 255) / 256); }

extern "C" int alofa_short_conv(void* out, int out_dtype, const void* h, int h_dtype, const float* w, const void* state, const int32_t* req_slot,
                                const int32_t* row_off, const int32_t* req_of_row, int rows, int width, int taps, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && width > 0 && taps >= 1 && taps - 1 <= kMaxKeep, "short_conv: bad sizes (rows=%d width=%d taps=%d, at most %d taps)", rows, width, taps, kMaxKeep + 1);
  ALOFA_REQUIRE(!exact || (out_dtype == kF32 && h_dtype == kF32), "short_conv: the exact path is float32");
  if (rows == 0) return 0;
  const unsigned grid = blocks_of(static_cast<int64_t>(rows) * width);
#define ALOFA_CONV(TO, TI, ACC) short_conv_kernel<TO, TI, ACC><<<grid, 256, 0, stream>>>(static_cast<TO*>(out), static_cast<const TI*>(h), w, static_cast<const TI*>(state), req_slot, row_off, req_of_row, rows, width, taps)
  if (exact) ALOFA_CONV(float, float, double);
  else if (out_dtype == kF32 && h_dtype == kF32) ALOFA_CONV(float, float, float);
  else if (out_dtype == kBF16 && h_dtype == kF32) ALOFA_CONV(bf16_t, float, float);
  else if (out_dtype == kBF16 && h_dtype == kBF16) ALOFA_CONV(bf16_t, bf16_t, float);
  else ALOFA_REQUIRE(false, "short_conv: no such pair of types (out=%d in=%d)", out_dtype, h_dtype);
#undef ALOFA_CONV
  return check_launch("short_conv");
}

extern "C" int alofa_keep_last_rows(void* state, const void* h, int dtype, const int32_t* req_slot, const int32_t* row_off, int requests, int width,
                                    int keep, hipStream_t stream) {
  ALOFA_REQUIRE(requests >= 0 && width > 0 && keep >= 0 && keep <= kMaxKeep, "keep_last_rows: bad sizes (requests=%d width=%d keep=%d)", requests, width, keep);
  if (requests == 0 || keep == 0) return 0;
  const unsigned grid = blocks_of(static_cast<int64_t>(requests) * width);
  if (dtype == kF32) keep_last_rows_kernel<float><<<grid, 256, 0, stream>>>(static_cast<float*>(state), static_cast<const float*>(h), req_slot, row_off, requests, width, keep);
  else keep_last_rows_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(state), static_cast<const bf16_t*>(h), req_slot, row_off, requests, width, keep);
  return check_launch("keep_last_rows");
}

extern "C" int alofa_shift_mix(void* out, const void* x, int dtype, const float* mu, const void* state, const int32_t* req_slot, const int32_t* row_off,
                               const int32_t* req_of_row, int rows, int width, int n_mixes, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && width > 0 && n_mixes >= 1, "shift_mix: bad sizes (rows=%d width=%d mixes=%d)", rows, width, n_mixes);
  if (rows == 0) return 0;
  const unsigned grid = blocks_of(static_cast<int64_t>(rows) * width);
  if (dtype == kF32) shift_mix_kernel<float><<<grid, 256, 0, stream>>>(static_cast<float*>(out), static_cast<const float*>(x), mu, static_cast<const float*>(state), req_slot, row_off, req_of_row, rows, width, n_mixes);
  else shift_mix_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(out), static_cast<const bf16_t*>(x), mu, static_cast<const bf16_t*>(state), req_slot, row_off, req_of_row, rows, width, n_mixes);
  return check_launch("shift_mix");
}

// Keys per thread and waves for a key size: four waves where that gives a share of 8, 16, 32 or 64 keys, more waves of 64 beyond.
static inline void recurrence_shape(int dk, int* kpt, int* waves) {
  const int quarter = (dk + 3) / 4;
  *kpt = quarter <= 8 ? 8 : quarter <= 16 ? 16 : quarter <= 32 ? 32 : 64;
  *waves = (dk + *kpt - 1) / *kpt;
}

extern "C" int alofa_linear_recurrence_lds_bytes(int dk, int chunk) {
  int kpt, waves;
  recurrence_shape(dk, &kpt, &waves);
  return chunk * (3 * waves * kpt + kWave + waves * kWave) * static_cast<int>(sizeof(float));
}

extern "C" int alofa_linear_recurrence(float* out, const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v, int64_t v_stride,
                                       int dtype, const float* decay_in, int64_t decay_stride, const float* decay_head, const float* bonus,
                                       float* state, const int32_t* req_slot, const int32_t* row_off, int requests, int heads, int dk, int dv,
                                       int decay_kind, float tau, float q_scale, float k_scale, int before_update, int chunk, hipStream_t stream) {
  ALOFA_REQUIRE(requests >= 0 && heads > 0 && dk > 0 && dk <= 512 && dv > 0, "linear_recurrence: bad sizes (requests=%d heads=%d dk=%d dv=%d; dk at most 512)", requests, heads, dk, dv);
  ALOFA_REQUIRE(decay_kind >= kDecayPerHead && decay_kind <= kDecayExpNegExp, "linear_recurrence: no such kind of decay (%d)", decay_kind);
  ALOFA_REQUIRE(decay_kind == kDecayPerHead ? decay_head != nullptr : decay_in != nullptr, "linear_recurrence: the decay's operand is absent");
  ALOFA_REQUIRE(decay_kind != kDecaySigmoidRoot || tau > 0.f, "linear_recurrence: tau must be positive");
  ALOFA_REQUIRE(chunk >= 1 && chunk <= 64, "linear_recurrence: rows per chunk lie in 1..64 (%d)", chunk);
  if (requests == 0) return 0;
  int kpt, waves;
  recurrence_shape(dk, &kpt, &waves);
  const int lds = alofa_linear_recurrence_lds_bytes(dk, chunk);
  ALOFA_REQUIRE(lds <= 64 * 1024, "linear_recurrence: a chunk of %d rows of %d keys does not fit LDS", chunk, dk);
  const dim3 grid((dv + kWave - 1) / kWave, heads, requests), block(waves * kWave);
  const float inv_tau = decay_kind == kDecaySigmoidRoot ? 1.f / tau : 0.f;
#define ALOFA_SCAN(T, KPT) linear_recurrence_kernel<T, KPT><<<grid, block, lds, stream>>>(out, static_cast<const T*>(q), q_stride, static_cast<const T*>(k), k_stride, \
    static_cast<const T*>(v), v_stride, decay_in, decay_stride, decay_head, bonus, state, req_slot, row_off, heads, dk, dv, decay_kind, inv_tau, q_scale, k_scale, before_update, chunk)
#define ALOFA_SCAN_T(T)                  \
  switch (kpt) {                         \
    case 8: ALOFA_SCAN(T, 8); break;     \
    case 16: ALOFA_SCAN(T, 16); break;   \
    case 32: ALOFA_SCAN(T, 32); break;   \
    default: ALOFA_SCAN(T, 64); break;   \
  }
  if (dtype == kF32) { ALOFA_SCAN_T(float) } else { ALOFA_SCAN_T(bf16_t) }
#undef ALOFA_SCAN_T
#undef ALOFA_SCAN
  return check_launch("linear_recurrence");
}
