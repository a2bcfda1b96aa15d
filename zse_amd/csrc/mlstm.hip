// Matrix-memory recurrence (mLSTM of xLSTM), one block per (request, head), token by token.
//
// Per head, with D query/key channels and E value channels, a state (S [D, E], n [D], m) that
// starts at zero and lives as floats in the request's state slot:
//
//   i_t = cap tanh((gi_t + bi) / cap)            f_t = logsigmoid(cap tanh((gf_t + bf) / cap))
//   m_t = max(f_t + m_(t-1), i_t)
//   S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T        (n_t likewise with k_t alone)
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6),      q_t already times D^(-1/2) here
//   out_t = o_t / sqrt(mean(o_t^2) + eps) * g[head] * sigmoid(z_t)
//
// q, k, v and z come from one product in the activation type; gi, gf are float.  Everything
// above is float.  The order of every sum depends on the token alone, so a request's values
// do not depend on how its tokens are cut into steps or on what else a step holds.
#include "common.h"
#include "packed_call.h"

extern "C" int zk_steplist_register(const char* name, int nargs, void* fn);
#define ZK_ENTER(fn) \
  static const int fn##_entered = zk_steplist_register(#fn, zk_packed::Call<fn>::nargs, (void*)zk_packed::Call<fn>::call);

#define MLSTM_THREADS 256

__device__ __forceinline__ float log_sigmoid(float x) {
  // min(x, 0) - log1p(exp(-|x|))
  return fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
}

__global__ __launch_bounds__(MLSTM_THREADS) void mlstm_kernel(
    const act_t* __restrict__ qkvz, int ld, const float* __restrict__ gates, const float* __restrict__ bias_i,
    const float* __restrict__ bias_f, const float* __restrict__ norm_w, float* __restrict__ state, int slot_words,
    int offset_words, const int* __restrict__ q_start, const int* __restrict__ slot_of_req, act_t* __restrict__ out,
    int H, int D, int E, float cap, float eps, float q_scale) {
  extern __shared__ float lds[];
  const int r = blockIdx.x, hd = blockIdx.y, tid = threadIdx.x;
  const int t0 = q_start[r], t1 = q_start[r + 1];
  if (t1 <= t0) return;                       // a padding request of a captured step
  float* S = lds;                              // [D][E]
  float* n = S + (size_t)D * E;                // [D]
  float* sq = n + D;                           // [D]
  float* sk = sq + D;                          // [D]
  float* sv = sk + D;                          // [E]
  float* part = sv + E;                        // [slices][E]
  float* red = part + MLSTM_THREADS;           // 17 + 1
  const size_t per_head = (size_t)D * E + D + 1;
  float* st = state + (size_t)slot_of_req[r] * slot_words + offset_words + (size_t)hd * per_head;
  for (int i = tid; i < D * E + D; i += MLSTM_THREADS) lds[i] = st[i];
  float m = st[(size_t)D * E + D];
  const int slices = MLSTM_THREADS / E > 0 ? MLSTM_THREADS / E : 1;     // E <= 256
  const int e = tid % E, sl = tid / E;
  const bool active = sl < slices;
  const int per = (D + slices - 1) / slices;
  const int d0 = sl * per, d1 = min(D, d0 + per);
  const float bi = bias_i[hd], bf = bias_f[hd];
  __syncthreads();
  for (int t = t0; t < t1; t++) {
    const act_t* row = qkvz + (size_t)t * ld;
    for (int d = tid; d < D; d += MLSTM_THREADS) {
      sq[d] = to_f32(row[(size_t)hd * D + d]) * q_scale;
      sk[d] = to_f32(row[(size_t)(H + hd) * D + d]);
    }
    for (int c = tid; c < E; c += MLSTM_THREADS) sv[c] = to_f32(row[(size_t)2 * H * D + (size_t)hd * E + c]);
    const float gi = cap * tanhf((gates[(size_t)t * 2 * H + hd] + bi) / cap);
    const float gf = log_sigmoid(cap * tanhf((gates[(size_t)t * 2 * H + H + hd] + bf) / cap));
    const float m_new = fmaxf(gf + m, gi);
    const float a = expf(gf + m - m_new), b = expf(gi - m_new);
    m = m_new;
    __syncthreads();
    // S and the numerator: a thread owns value channel e and a slice of the key channels
    if (active) {
      const float bv = b * sv[e];
      float acc = 0.f;
      for (int d = d0; d < d1; d++) {
        const float s = fmaf(a, S[(size_t)d * E + e], sk[d] * bv);
        S[(size_t)d * E + e] = s;
        acc = fmaf(s, sq[d], acc);
      }
      part[sl * E + e] = acc;
    }
    // n and n . q
    float nq = 0.f;
    for (int d = tid; d < D; d += MLSTM_THREADS) {
      const float v = fmaf(a, n[d], b * sk[d]);
      n[d] = v;
      nq = fmaf(v, sq[d], nq);
    }
    nq = block_sum(nq, red);              // syncs: part[] is complete after it
    const float den = fmaxf(fabsf(nq), expf(-m)) + 1e-6f;
    float o = 0.f;
    if (tid < E) {
      for (int s2 = 0; s2 < slices; s2++) o += part[s2 * E + tid];
      o = o / den;
    }
    const float ms = block_sum(tid < E ? o * o : 0.f, red) / (float)E;
    if (tid < E) {
      const size_t col = (size_t)hd * E + tid;
      const float z = to_f32(row[(size_t)2 * H * D + (size_t)H * E + col]);
      const float y = o / sqrtf(ms + eps) * norm_w[col] * (1.0f / (1.0f + expf(-z)));
      out[(size_t)t * H * E + col] = from_f32<act_t>(y);
    }
    __syncthreads();
  }
  for (int i = tid; i < D * E + D; i += MLSTM_THREADS) st[i] = lds[i];
  if (tid == 0) st[(size_t)D * E + D] = m;
}

extern "C" {

size_t zk_mlstm_state_bytes(int H, int D, int E) { return (size_t)H * ((size_t)D * E + D + 1) * 4; }

// qkvz: [T, ld] activations, a row holding q [H, D] | k [H, D] | v [H, E] | z [H, E];
// gates: float [T, 2H] (input gates, then forget gates, before bias and cap); out: [T, H * E].
int zk_mlstm(const void* qkvz, int ld, const float* gates, const float* bias_i, const float* bias_f,
             const float* norm_w, float* state, int slot_words, int offset_words, const int* q_start,
             const int* slot_of_req, void* out, int R, int H, int D, int E, float cap, float eps, void* stream) {
  ZK_REQUIRE(R >= 0 && H > 0 && H <= 65535 && D > 0 && E > 0, "zk_mlstm: bad sizes");
  ZK_REQUIRE(E <= MLSTM_THREADS, "zk_mlstm: more than 256 value channels a head are not supported");
  ZK_REQUIRE(ld >= 2 * H * (D + E), "zk_mlstm: rows too short");
  ZK_REQUIRE(cap > 0.f, "zk_mlstm: the gates' cap must be positive");
  ZK_REQUIRE((size_t)slot_words * 4 >= (size_t)offset_words * 4 + zk_mlstm_state_bytes(H, D, E),
             "zk_mlstm: the state does not fit its slot");
  if (R == 0) return 0;
  const size_t lds = ((size_t)D * E + 3 * D + E + MLSTM_THREADS + 32) * 4;
  ZK_REQUIRE(lds <= 160 * 1024, "zk_mlstm: a head's state does not fit the local memory");
  if (lds > 48 * 1024) {
    static size_t raised = 0;
    if (lds > raised) {
      hipFuncSetAttribute((const void*)mlstm_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      raised = lds;
    }
  }
  dim3 grid(R, H);
  mlstm_kernel<<<grid, MLSTM_THREADS, lds, (hipStream_t)stream>>>(
      (const act_t*)qkvz, ld, gates, bias_i, bias_f, norm_w, state, slot_words, offset_words, q_start, slot_of_req,
      (act_t*)out, H, D, E, cap, eps, 1.0f / sqrtf((float)D));
  return zk_launch_status("zk_mlstm");
}

}  // extern "C"

ZK_ENTER(zk_mlstm)
