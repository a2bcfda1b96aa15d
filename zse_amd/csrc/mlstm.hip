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

// DIRECT: S stays in the state slot and every element is read, renewed and written back once per
// token, many loads in flight (steps of single tokens, where staging S through the local memory
// would only add two passes); else S is staged for the step's tokens.  The same arithmetic in
// the same order either way.
template <bool DIRECT>
__global__ __launch_bounds__(MLSTM_THREADS) void mlstm_kernel(
    const act_t* __restrict__ qkvz, int ld, const float* __restrict__ gates, const float* __restrict__ bias_i,
    const float* __restrict__ bias_f, const float* __restrict__ norm_w, float* __restrict__ state, int slot_words,
    int offset_words, const int* __restrict__ q_start, const int* __restrict__ slot_of_req, act_t* __restrict__ out,
    int H, int D, int E, float cap, float eps, float q_scale) {
  extern __shared__ float lds[];
  const int r = blockIdx.x, hd = blockIdx.y, tid = threadIdx.x;
  const int t0 = q_start[r], t1 = q_start[r + 1];
  if (t1 <= t0) return;                       // a padding request of a captured step
  const size_t per_head = (size_t)D * E + D + 1;
  float* st = state + (size_t)slot_of_req[r] * slot_words + offset_words + (size_t)hd * per_head;
  float* S = DIRECT ? st : lds;                // [D][E]
  float* n = DIRECT ? lds : lds + (size_t)D * E;      // [D]
  float* sq = n + D;                           // [D]
  float* sk = sq + D;                          // [D]
  float* sv = sk + D;                          // [E]
  float* part = sv + E;                        // [slices][E]
  float* red = part + MLSTM_THREADS;           // 17 + 1
  if (DIRECT) {
    for (int d = tid; d < D; d += MLSTM_THREADS) n[d] = st[(size_t)D * E + d];
  } else {
    for (int i = tid; i < D * E + D; i += MLSTM_THREADS) lds[i] = st[i];
  }
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
      // eight elements of S are asked for before the first of them is written back: the loads
      // of a thread's column are then in flight together (the sums keep their order)
      for (int d = d0; d < d1; d += 8) {
        float old[8];
#pragma unroll
        for (int x = 0; x < 8; x++) old[x] = d + x < d1 ? S[(size_t)(d + x) * E + e] : 0.f;
#pragma unroll
        for (int x = 0; x < 8; x++)
          if (d + x < d1) {
            const float s = fmaf(a, old[x], sk[d + x] * bv);
            S[(size_t)(d + x) * E + e] = s;
            acc = fmaf(s, sq[d + x], acc);
          }
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
  if (DIRECT) {
    for (int d = tid; d < D; d += MLSTM_THREADS) st[(size_t)D * E + d] = n[d];
  } else {
    for (int i = tid; i < D * E + D; i += MLSTM_THREADS) st[i] = lds[i];
  }
  if (tid == 0) st[(size_t)D * E + D] = m;
}

// ---- the same recurrence over chunks of L tokens, for steps that bring portions of prompts.
//
// Inside a chunk that starts from the state (S0, n0, m0), with F_j the sum of the forget gates up
// to token j of the chunk and a_s = i_s - F_s:
//
//   M_j = max(m0, max_{s<=j} a_s)                     m_j = F_j + M_j
//   P_js = (q_j . k_s) exp(a_s - M_j)  for s <= j     g_j = exp(m0 - M_j)
//   S_j^T q_j = g_j S0^T q_j + sum_s P_js v_s         n_j . q_j = g_j n0 . q_j + sum_s P_js
//
// which is the token-by-token recurrence written out (every exponent is <= 0).  At the chunk's
// last token the state becomes g S0 + sum_s exp(a_s - M) k_s v_s^T.  So a chunk is four small
// matrix products (q k^T, P v, q S0, k^T v) instead of L dependent steps.  A block owns 32
// value channels of a head: the recurrence never mixes value channels, only the norm over a
// head's read-out does, and that (with the gain and the output gate) is left to a second
// kernel, which also stores the new n and m: every block of a head computes them, none may
// store them while another still reads the old ones.
#define MLSTM_EC 32

__device__ __forceinline__ void load8(const float* p, float v[8]) {
  const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
  v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
}
__device__ __forceinline__ void load8(const __bf16* p, float v[8]) {
  typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
  const bf8 a = *(const bf8*)p;
#pragma unroll
  for (int x = 0; x < 8; x++) v[x] = (float)a[x];
}

template <int L>
__global__ __launch_bounds__(MLSTM_THREADS) void mlstm_chunk_kernel(
    const act_t* __restrict__ qkvz, int ld, const float* __restrict__ gates, const float* __restrict__ bias_i,
    const float* __restrict__ bias_f, float* __restrict__ state, int slot_words, int offset_words,
    const int* __restrict__ q_start, const int* __restrict__ slot_of_req, float* __restrict__ o_raw,
    float* __restrict__ nm_new, int H, int D, int E, float cap, float q_scale) {
  constexpr int EC = MLSTM_EC;
  constexpr int TP = L / 16;
  extern __shared__ float lds[];
  const int r = blockIdx.x, hd = blockIdx.y, e0 = blockIdx.z * EC, tid = threadIdx.x;
  const int t0 = q_start[r], t1 = q_start[r + 1];
  if (t1 <= t0) return;
  const int DP = D + 1, LP = L + 1;
  float* Ss = lds;                      // [D][EC]   this block's columns of S
  float* ns = Ss + (size_t)D * EC;      // [D]
  float* Qs = ns + D;                   // [L][DP]
  float* Ks = Qs + (size_t)L * DP;      // [L][DP]
  float* Vs = Ks + (size_t)L * DP;      // [L][EC]
  float* Ps = Vs + (size_t)L * EC;      // [L][LP]
  float* ga = Ps + (size_t)L * LP;      // a_s, then (after the scan) i_s - F_s
  float* gM = ga + L;                   // M_j
  float* gF = gM + L;                   // f_s, then F_j
  float* gden = gF + L;                 // denominators
  float* gw = gden + L;                 // exp(a_s - M_last)
  const size_t per_head = (size_t)D * E + D + 1;
  float* st = state + (size_t)slot_of_req[r] * slot_words + offset_words + (size_t)hd * per_head;
  for (int i = tid; i < D * EC; i += MLSTM_THREADS) {
    const int d = i / EC, e = e0 + i % EC;
    Ss[i] = e < E ? st[(size_t)d * E + e] : 0.f;
  }
  for (int d = tid; d < D; d += MLSTM_THREADS) ns[d] = st[(size_t)D * E + d];
  float m_prev = st[(size_t)D * E + D];
  const float bi = bias_i[hd], bf = bias_f[hd];
  const bool vec8 = D % 8 == 0 && ld % 8 == 0 && (uintptr_t)qkvz % 16 == 0;
  __syncthreads();
  for (int c0 = t0; c0 < t1; c0 += L) {
    const int Lc = min(L, t1 - c0);
    if (vec8) {      // eight channels a load
      const int D8 = D / 8;
      for (int i = tid; i < L * D8; i += MLSTM_THREADS) {
        const int j = i / D8, d = (i % D8) * 8;
        float q[8] = {}, k[8] = {};
        if (j < Lc) {
          const act_t* row = qkvz + (size_t)(c0 + j) * ld;
          load8(row + (size_t)hd * D + d, q);
          load8(row + (size_t)(H + hd) * D + d, k);
        }
#pragma unroll
        for (int x = 0; x < 8; x++) {
          Qs[j * DP + d + x] = q[x] * q_scale;
          Ks[j * DP + d + x] = k[x];
        }
      }
    } else {
      for (int i = tid; i < L * D; i += MLSTM_THREADS) {
        const int j = i / D, d = i % D;
        float q = 0.f, k = 0.f;
        if (j < Lc) {
          const act_t* row = qkvz + (size_t)(c0 + j) * ld;
          q = to_f32(row[(size_t)hd * D + d]) * q_scale;
          k = to_f32(row[(size_t)(H + hd) * D + d]);
        }
        Qs[j * DP + d] = q;
        Ks[j * DP + d] = k;
      }
    }
    for (int i = tid; i < L * EC; i += MLSTM_THREADS) {
      const int j = i / EC, e = e0 + i % EC;
      Vs[i] = (j < Lc && e < E) ? to_f32(qkvz[(size_t)(c0 + j) * ld + (size_t)2 * H * D + (size_t)hd * E + e]) : 0.f;
    }
    if (tid < Lc) {
      const size_t t = c0 + tid;
      ga[tid] = cap * tanhf((gates[t * 2 * H + hd] + bi) / cap);
      gF[tid] = log_sigmoid(cap * tanhf((gates[t * 2 * H + H + hd] + bf) / cap));
    }
    __syncthreads();
    if (tid < ZSE_WAVE) {      // running sums of the forget gates and running maxima of a, over one wave (L <= 64)
      const int j = tid;
      float F = j < Lc ? gF[j] : 0.f;
#pragma unroll
      for (int o = 1; o < ZSE_WAVE; o <<= 1) {
        const float up = __shfl_up(F, o, ZSE_WAVE);
        if (j >= o) F += up;
      }
      const float a = j < Lc ? ga[j] - F : -INFINITY;
      float M = a;
#pragma unroll
      for (int o = 1; o < ZSE_WAVE; o <<= 1) {
        const float up = __shfl_up(M, o, ZSE_WAVE);
        if (j >= o) M = fmaxf(M, up);
      }
      if (j < L) {
        ga[j] = a;
        gM[j] = fmaxf(M, m_prev);
        gF[j] = F;
      }
    }
    __syncthreads();
    {  // P
      // rows pj + 16 a, columns ps + 16 b: neighbouring lanes read neighbouring rows of K
      const int pj = tid / 16, ps = tid % 16;
      float acc[TP][TP] = {};
      for (int d = 0; d < D; d++) {
        float q[TP], k[TP];
#pragma unroll
        for (int x = 0; x < TP; x++) {
          q[x] = Qs[(pj + 16 * x) * DP + d];
          k[x] = Ks[(ps + 16 * x) * DP + d];
        }
#pragma unroll
        for (int a = 0; a < TP; a++)
#pragma unroll
          for (int b = 0; b < TP; b++) acc[a][b] = fmaf(q[a], k[b], acc[a][b]);
      }
#pragma unroll
      for (int a = 0; a < TP; a++)
#pragma unroll
        for (int b = 0; b < TP; b++) {
          const int j = pj + 16 * a, s2 = ps + 16 * b;
          Ps[j * LP + s2] = (s2 <= j && j < Lc) ? acc[a][b] * expf(ga[s2] - gM[j]) : 0.f;
        }
    }
    __syncthreads();
    if (tid < L) {  // denominators
      const int j = tid;
      float nq = 0.f;
      for (int d = 0; d < D; d++) nq = fmaf(ns[d], Qs[j * DP + d], nq);
      nq *= expf(m_prev - gM[j]);
      for (int s2 = 0; s2 <= j; s2++) nq += Ps[j * LP + s2];
      gden[j] = fmaxf(fabsf(nq), expf(-(gF[j] + gM[j]))) + 1e-6f;
      gw[j] = j < Lc ? expf(ga[j] - gM[Lc - 1]) : 0.f;
    }
    {  // read-out: TP rows, columns ec, ec + 1
      const int ec = (tid % 16) * 2, rg = tid / 16;        // rows rg + 16 a
      float acc[TP][2] = {};
      for (int d = 0; d < D; d++) {
        const float s0 = Ss[d * EC + ec], s1 = Ss[d * EC + ec + 1];
#pragma unroll
        for (int a = 0; a < TP; a++) {
          const float q = Qs[(rg + 16 * a) * DP + d];
          acc[a][0] = fmaf(q, s0, acc[a][0]);
          acc[a][1] = fmaf(q, s1, acc[a][1]);
        }
      }
#pragma unroll
      for (int a = 0; a < TP; a++) {
        const float g = expf(m_prev - gM[rg + 16 * a]);
        acc[a][0] *= g;
        acc[a][1] *= g;
      }
      for (int s2 = 0; s2 < Lc; s2++) {
        const float v0 = Vs[s2 * EC + ec], v1 = Vs[s2 * EC + ec + 1];
#pragma unroll
        for (int a = 0; a < TP; a++) {
          const float p = Ps[(rg + 16 * a) * LP + s2];
          acc[a][0] = fmaf(p, v0, acc[a][0]);
          acc[a][1] = fmaf(p, v1, acc[a][1]);
        }
      }
      __syncthreads();          // the denominators are there; every read of Vs is done
#pragma unroll
      for (int a = 0; a < TP; a++) {
        const int j = rg + 16 * a;
        if (j < Lc) {
          float* o = o_raw + ((size_t)(c0 + j) * H + hd) * E;
          if (e0 + ec < E) o[e0 + ec] = acc[a][0] / gden[j];
          if (e0 + ec + 1 < E) o[e0 + ec + 1] = acc[a][1] / gden[j];
        }
      }
    }
    // the state after the chunk's last token
    const float M_last = gM[Lc - 1];
    const float g_last = expf(m_prev - M_last);
    const float m_next = gF[Lc - 1] + M_last;
    for (int i = tid; i < L * EC; i += MLSTM_THREADS) Vs[i] *= gw[i / EC];
    for (int d = tid; d < D; d += MLSTM_THREADS) {
      float acc = 0.f;
      for (int s2 = 0; s2 < Lc; s2++) acc = fmaf(gw[s2], Ks[s2 * DP + d], acc);
      ns[d] = fmaf(g_last, ns[d], acc);
    }
    __syncthreads();
    {
      const int ec = (tid % 16) * 2, dg = (tid / 16) * 4;
      for (int db = 0; db < D; db += 64) {
        float acc[4][2] = {};
        const int d = db + dg;
        for (int s2 = 0; s2 < Lc; s2++) {
          const float v0 = Vs[s2 * EC + ec], v1 = Vs[s2 * EC + ec + 1];
#pragma unroll
          for (int a = 0; a < 4; a++) {
            const float k = d + a < D ? Ks[s2 * DP + d + a] : 0.f;
            acc[a][0] = fmaf(k, v0, acc[a][0]);
            acc[a][1] = fmaf(k, v1, acc[a][1]);
          }
        }
#pragma unroll
        for (int a = 0; a < 4; a++)
          if (d + a < D) {
            float* sp = Ss + (size_t)(d + a) * EC + ec;
            sp[0] = fmaf(g_last, sp[0], acc[a][0]);
            sp[1] = fmaf(g_last, sp[1], acc[a][1]);
          }
      }
    }
    m_prev = m_next;
    __syncthreads();
  }
  for (int i = tid; i < D * EC; i += MLSTM_THREADS) {
    const int d = i / EC, e = e0 + i % EC;
    if (e < E) st[(size_t)d * E + e] = Ss[i];
  }
  if (blockIdx.z == 0) {
    float* nm = nm_new + ((size_t)r * H + hd) * (D + 1);
    for (int d = tid; d < D; d += MLSTM_THREADS) nm[d] = ns[d];
    if (tid == 0) nm[D] = m_prev;
  }
}

// The read-out's norm over each head, gain and output gate; the block of a request's last
// token also stores the head's new n and m.
__global__ __launch_bounds__(64) void mlstm_finish_kernel(
    const float* __restrict__ o_raw, const act_t* __restrict__ qkvz, int ld, const float* __restrict__ norm_w,
    const float* __restrict__ nm_new, float* __restrict__ state, int slot_words, int offset_words,
    const int* __restrict__ req_of_token, const int* __restrict__ q_start, const int* __restrict__ slot_of_req,
    act_t* __restrict__ out, int H, int D, int E, float eps) {
  const int t = blockIdx.x, hd = blockIdx.y, lane = threadIdx.x;
  const float* o = o_raw + ((size_t)t * H + hd) * E;
  float ss = 0.f;
  for (int e = lane; e < E; e += 64) ss = fmaf(o[e], o[e], ss);
  const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)E + eps);
  const act_t* z = qkvz + (size_t)t * ld + (size_t)2 * H * D + (size_t)H * E + (size_t)hd * E;
  for (int e = lane; e < E; e += 64) {
    const float y = o[e] * inv * norm_w[(size_t)hd * E + e] * (1.0f / (1.0f + expf(-to_f32(z[e]))));
    out[((size_t)t * H + hd) * E + e] = from_f32<act_t>(y);
  }
  if (nm_new == nullptr) return;
  const int r = req_of_token[t];
  if (t == q_start[r + 1] - 1) {
    float* st = state + (size_t)slot_of_req[r] * slot_words + offset_words + (size_t)hd * ((size_t)D * E + D + 1) + (size_t)D * E;
    const float* nm = nm_new + ((size_t)r * H + hd) * (D + 1);
    for (int d = lane; d <= D; d += 64) st[d] = nm[d];
  }
}

// ---- the chunks of long portions side by side, in three launches.
//
// The chunk kernel above walks a request's chunks one after the other, since each starts from the
// state the one before left: a head keeps at most a few blocks busy however long the portion.
// What a chunk adds to the state does not depend on that state, though:
//
//   local  (every chunk at once):   A = max_s a_s,  U = sum_s exp(a_s - A) k_s v_s^T,  u likewise,  F = F_L
//   scan   (chunk after chunk, one multiply-add per element of the state):
//          M = max(m0, A),  S0' = exp(m0 - M) S0 + exp(A - M) U,  m0' = F + M;   S0, n0, m0 of every chunk are kept
//   output (every chunk at once):   the read-out of the chunk kernel from the kept S0, n0, m0
//
// Chunks are numbered through the step's requests (request r has ceil(n_r / L) of them); a block
// finds its request by walking q_start.  U is stored where the scan then leaves S0 of that chunk.
__device__ __forceinline__ bool mlstm_find_chunk(const int* __restrict__ q_start, int R, int L, int x, int& r, int& c0,
                                                 int& Lc) {
  int acc = 0;
  for (r = 0; r < R; r++) {
    const int t0 = q_start[r], n = q_start[r + 1] - t0;
    const int nc = (n + L - 1) / L;
    if (x < acc + nc) {
      c0 = t0 + (x - acc) * L;
      Lc = min(L, t0 + n - c0);
      return true;
    }
    acc += nc;
  }
  return false;
}

// Loads a chunk's k (and q) rows and its slice of v into the local memory, zero beyond Lc.
template <int L, bool WITH_Q>
__device__ __forceinline__ void mlstm_load_chunk(const act_t* __restrict__ qkvz, int ld, int c0, int Lc, int hd, int e0, int H,
                                                 int D, int E, float q_scale, float* Qs, float* Ks, float* Vs) {
  const int tid = threadIdx.x, DP = D + 1;
  const bool vec8 = D % 8 == 0 && ld % 8 == 0 && (uintptr_t)qkvz % 16 == 0;
  if (vec8) {
    const int D8 = D / 8;
    for (int i = tid; i < L * D8; i += MLSTM_THREADS) {
      const int j = i / D8, d = (i % D8) * 8;
      float q[8] = {}, k[8] = {};
      if (j < Lc) {
        const act_t* row = qkvz + (size_t)(c0 + j) * ld;
        if (WITH_Q) load8(row + (size_t)hd * D + d, q);
        load8(row + (size_t)(H + hd) * D + d, k);
      }
#pragma unroll
      for (int x = 0; x < 8; x++) {
        if (WITH_Q) Qs[j * DP + d + x] = q[x] * q_scale;
        Ks[j * DP + d + x] = k[x];
      }
    }
  } else {
    for (int i = tid; i < L * D; i += MLSTM_THREADS) {
      const int j = i / D, d = i % D;
      float q = 0.f, k = 0.f;
      if (j < Lc) {
        const act_t* row = qkvz + (size_t)(c0 + j) * ld;
        if (WITH_Q) q = to_f32(row[(size_t)hd * D + d]) * q_scale;
        k = to_f32(row[(size_t)(H + hd) * D + d]);
      }
      if (WITH_Q) Qs[j * DP + d] = q;
      Ks[j * DP + d] = k;
    }
  }
  for (int i = tid; i < L * MLSTM_EC; i += MLSTM_THREADS) {
    const int j = i / MLSTM_EC, e = e0 + i % MLSTM_EC;
    Vs[i] = (j < Lc && e < E) ? to_f32(qkvz[(size_t)(c0 + j) * ld + (size_t)2 * H * D + (size_t)hd * E + e]) : 0.f;
  }
}

template <int L>
__global__ __launch_bounds__(MLSTM_THREADS) void mlstm_local_kernel(
    const act_t* __restrict__ qkvz, int ld, const float* __restrict__ gates, const float* __restrict__ bias_i,
    const float* __restrict__ bias_f, const int* __restrict__ q_start, float* __restrict__ Uw, float* __restrict__ uw,
    float* __restrict__ af, int R, int H, int D, int E, float cap) {
  constexpr int EC = MLSTM_EC;
  extern __shared__ float lds[];
  const int x = blockIdx.x, hd = blockIdx.y, e0 = blockIdx.z * EC, tid = threadIdx.x;
  int r, c0, Lc;
  if (!mlstm_find_chunk(q_start, R, L, x, r, c0, Lc)) return;
  const int DP = D + 1;
  float* Ks = lds;                       // [L][DP]
  float* Vs = Ks + (size_t)L * DP;       // [L][EC]
  float* ga = Vs + (size_t)L * EC;
  float* gF = ga + L;
  float* gw = gF + L;
  mlstm_load_chunk<L, false>(qkvz, ld, c0, Lc, hd, e0, H, D, E, 0.f, nullptr, Ks, Vs);
  if (tid < ZSE_WAVE) {
    const int j = tid;
    float F = 0.f, gi = 0.f;
    if (j < Lc) {
      const size_t t = c0 + j;
      gi = cap * tanhf((gates[t * 2 * H + hd] + bias_i[hd]) / cap);
      F = log_sigmoid(cap * tanhf((gates[t * 2 * H + H + hd] + bias_f[hd]) / cap));
    }
#pragma unroll
    for (int o = 1; o < ZSE_WAVE; o <<= 1) {
      const float up = __shfl_up(F, o, ZSE_WAVE);
      if (j >= o) F += up;
    }
    const float a = j < Lc ? gi - F : -INFINITY;
    const float A = wave_max(a);
    if (j < L) gw[j] = j < Lc ? expf(a - A) : 0.f;
    if (j == Lc - 1 && blockIdx.z == 0) {
      af[((size_t)x * H + hd) * 2] = A;
      af[((size_t)x * H + hd) * 2 + 1] = F;
    }
  }
  __syncthreads();
  for (int i = tid; i < L * EC; i += MLSTM_THREADS) Vs[i] *= gw[i / EC];
  if (blockIdx.z == 0)
    for (int d = tid; d < D; d += MLSTM_THREADS) {
      float acc = 0.f;
      for (int s2 = 0; s2 < Lc; s2++) acc = fmaf(gw[s2], Ks[s2 * DP + d], acc);
      uw[((size_t)x * H + hd) * D + d] = acc;
    }
  __syncthreads();
  float* U = Uw + ((size_t)x * H + hd) * D * E;
  const int ec = (tid % 16) * 2, dg = (tid / 16) * 4;
  for (int db = 0; db < D; db += 64) {
    float acc[4][2] = {};
    const int d = db + dg;
    for (int s2 = 0; s2 < Lc; s2++) {
      const float v0 = Vs[s2 * EC + ec], v1 = Vs[s2 * EC + ec + 1];
#pragma unroll
      for (int a = 0; a < 4; a++) {
        const float k = d + a < D ? Ks[s2 * DP + d + a] : 0.f;
        acc[a][0] = fmaf(k, v0, acc[a][0]);
        acc[a][1] = fmaf(k, v1, acc[a][1]);
      }
    }
#pragma unroll
    for (int a = 0; a < 4; a++)
      if (d + a < D) {
        if (e0 + ec < E) U[(size_t)(d + a) * E + e0 + ec] = acc[a][0];
        if (e0 + ec + 1 < E) U[(size_t)(d + a) * E + e0 + ec + 1] = acc[a][1];
      }
  }
}

// One thread per element of a head's state (S, then n, then one more thread that keeps m).
__global__ __launch_bounds__(MLSTM_THREADS) void mlstm_scan_kernel(
    float* __restrict__ state, int slot_words, int offset_words, const int* __restrict__ q_start,
    const int* __restrict__ slot_of_req, float* __restrict__ Uw, float* __restrict__ uw, const float* __restrict__ af,
    float* __restrict__ mprev, int L, int H, int D, int E) {
  const int r = blockIdx.x, hd = blockIdx.y;
  const int idx = blockIdx.z * MLSTM_THREADS + threadIdx.x;
  const int DE = D * E;
  if (idx > DE + D) return;
  const int t0 = q_start[r], n = q_start[r + 1] - t0;
  if (n <= 0) return;
  int first = 0;
  for (int r2 = 0; r2 < r; r2++) first += (q_start[r2 + 1] - q_start[r2] + L - 1) / L;
  const int nc = (n + L - 1) / L;
  float* st = state + (size_t)slot_of_req[r] * slot_words + offset_words + (size_t)hd * ((size_t)DE + D + 1);
  float m = st[DE + D];
  float val = idx < DE + D ? st[idx] : 0.f;
  for (int ci = 0; ci < nc; ci++) {
    const size_t at = (size_t)(first + ci) * H + hd;
    const float A = af[at * 2], F = af[at * 2 + 1];
    const float M = fmaxf(m, A);
    if (idx < DE + D) {
      float* p = idx < DE ? Uw + at * DE + idx : uw + at * D + (idx - DE);
      const float U = *p;
      *p = val;                                   // the state this chunk starts from
      val = fmaf(expf(m - M), val, expf(A - M) * U);
    } else {
      mprev[at] = m;
    }
    m = F + M;
  }
  st[idx] = idx < DE + D ? val : m;
}

template <int L>
__global__ __launch_bounds__(MLSTM_THREADS) void mlstm_output_kernel(
    const act_t* __restrict__ qkvz, int ld, const float* __restrict__ gates, const float* __restrict__ bias_i,
    const float* __restrict__ bias_f, const int* __restrict__ q_start, const float* __restrict__ Sw,
    const float* __restrict__ nw, const float* __restrict__ mprev, float* __restrict__ o_raw, int R, int H, int D, int E,
    float cap, float q_scale) {
  constexpr int EC = MLSTM_EC;
  constexpr int TP = L / 16;
  extern __shared__ float lds[];
  const int x = blockIdx.x, hd = blockIdx.y, e0 = blockIdx.z * EC, tid = threadIdx.x;
  int r, c0, Lc;
  if (!mlstm_find_chunk(q_start, R, L, x, r, c0, Lc)) return;
  const int DP = D + 1, LP = L + 1;
  float* Ss = lds;
  float* ns = Ss + (size_t)D * EC;
  float* Qs = ns + D;
  float* Ks = Qs + (size_t)L * DP;
  float* Vs = Ks + (size_t)L * DP;
  float* Ps = Vs + (size_t)L * EC;
  float* ga = Ps + (size_t)L * LP;
  float* gM = ga + L;
  float* gF = gM + L;
  float* gden = gF + L;
  const size_t at = (size_t)x * H + hd;
  const float* S0 = Sw + at * D * E;
  for (int i = tid; i < D * EC; i += MLSTM_THREADS) {
    const int d = i / EC, e = e0 + i % EC;
    Ss[i] = e < E ? S0[(size_t)d * E + e] : 0.f;
  }
  for (int d = tid; d < D; d += MLSTM_THREADS) ns[d] = nw[at * D + d];
  const float m_prev = mprev[at];
  mlstm_load_chunk<L, true>(qkvz, ld, c0, Lc, hd, e0, H, D, E, q_scale, Qs, Ks, Vs);
  if (tid < ZSE_WAVE) {
    const int j = tid;
    float F = 0.f, gi = 0.f;
    if (j < Lc) {
      const size_t t = c0 + j;
      gi = cap * tanhf((gates[t * 2 * H + hd] + bias_i[hd]) / cap);
      F = log_sigmoid(cap * tanhf((gates[t * 2 * H + H + hd] + bias_f[hd]) / cap));
    }
#pragma unroll
    for (int o = 1; o < ZSE_WAVE; o <<= 1) {
      const float up = __shfl_up(F, o, ZSE_WAVE);
      if (j >= o) F += up;
    }
    const float a = j < Lc ? gi - F : -INFINITY;
    float M = a;
#pragma unroll
    for (int o = 1; o < ZSE_WAVE; o <<= 1) {
      const float up = __shfl_up(M, o, ZSE_WAVE);
      if (j >= o) M = fmaxf(M, up);
    }
    if (j < L) {
      ga[j] = a;
      gM[j] = fmaxf(M, m_prev);
      gF[j] = F;
    }
  }
  __syncthreads();
  {
    const int pj = tid / 16, ps = tid % 16;
    float acc[TP][TP] = {};
    for (int d = 0; d < D; d++) {
      float q[TP], k[TP];
#pragma unroll
      for (int y = 0; y < TP; y++) {
        q[y] = Qs[(pj + 16 * y) * DP + d];
        k[y] = Ks[(ps + 16 * y) * DP + d];
      }
#pragma unroll
      for (int a = 0; a < TP; a++)
#pragma unroll
        for (int b = 0; b < TP; b++) acc[a][b] = fmaf(q[a], k[b], acc[a][b]);
    }
#pragma unroll
    for (int a = 0; a < TP; a++)
#pragma unroll
      for (int b = 0; b < TP; b++) {
        const int j = pj + 16 * a, s2 = ps + 16 * b;
        Ps[j * LP + s2] = (s2 <= j && j < Lc) ? acc[a][b] * expf(ga[s2] - gM[j]) : 0.f;
      }
  }
  __syncthreads();
  if (tid < L) {
    const int j = tid;
    float nq = 0.f;
    for (int d = 0; d < D; d++) nq = fmaf(ns[d], Qs[j * DP + d], nq);
    nq *= expf(m_prev - gM[j]);
    for (int s2 = 0; s2 <= j; s2++) nq += Ps[j * LP + s2];
    gden[j] = fmaxf(fabsf(nq), expf(-(gF[j] + gM[j]))) + 1e-6f;
  }
  const int ec = (tid % 16) * 2, rg = tid / 16;
  float acc[TP][2] = {};
  for (int d = 0; d < D; d++) {
    const float s0 = Ss[d * EC + ec], s1 = Ss[d * EC + ec + 1];
#pragma unroll
    for (int a = 0; a < TP; a++) {
      const float q = Qs[(rg + 16 * a) * DP + d];
      acc[a][0] = fmaf(q, s0, acc[a][0]);
      acc[a][1] = fmaf(q, s1, acc[a][1]);
    }
  }
#pragma unroll
  for (int a = 0; a < TP; a++) {
    const float g = expf(m_prev - gM[rg + 16 * a]);
    acc[a][0] *= g;
    acc[a][1] *= g;
  }
  for (int s2 = 0; s2 < Lc; s2++) {
    const float v0 = Vs[s2 * EC + ec], v1 = Vs[s2 * EC + ec + 1];
#pragma unroll
    for (int a = 0; a < TP; a++) {
      const float p = Ps[(rg + 16 * a) * LP + s2];
      acc[a][0] = fmaf(p, v0, acc[a][0]);
      acc[a][1] = fmaf(p, v1, acc[a][1]);
    }
  }
  __syncthreads();
#pragma unroll
  for (int a = 0; a < TP; a++) {
    const int j = rg + 16 * a;
    if (j < Lc) {
      float* o = o_raw + ((size_t)(c0 + j) * H + hd) * E;
      if (e0 + ec < E) o[e0 + ec] = acc[a][0] / gden[j];
      if (e0 + ec + 1 < E) o[e0 + ec + 1] = acc[a][1] / gden[j];
    }
  }
}

static size_t mlstm_chunk_lds(int L, int D) {
  return ((size_t)D * MLSTM_EC + D + (size_t)2 * L * (D + 1) + (size_t)L * MLSTM_EC + (size_t)L * (L + 1) + 5 * L + 8) * 4;
}

template <int L>
static int mlstm_chunk_launch(const void* qkvz, int ld, const float* gates, const float* bias_i, const float* bias_f,
                              float* state, int slot_words, int offset_words, const int* q_start,
                              const int* slot_of_req, float* o_raw, float* nm_new, int R, int H, int D, int E,
                              float cap, hipStream_t stream) {
  const size_t lds = mlstm_chunk_lds(L, D);
  static size_t raised = 0;
  if (lds > 48 * 1024 && lds > raised) {
    hipFuncSetAttribute((const void*)mlstm_chunk_kernel<L>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    raised = lds;
  }
  dim3 grid(R, H, (E + MLSTM_EC - 1) / MLSTM_EC);
  mlstm_chunk_kernel<L><<<grid, MLSTM_THREADS, lds, stream>>>((const act_t*)qkvz, ld, gates, bias_i, bias_f, state,
                                                              slot_words, offset_words, q_start, slot_of_req, o_raw,
                                                              nm_new, H, D, E, cap, 1.0f / sqrtf((float)D));
  return zk_launch_status("zk_mlstm_chunked");
}

extern "C" {

size_t zk_mlstm_state_bytes(int H, int D, int E) { return (size_t)H * ((size_t)D * E + D + 1) * 4; }

// qkvz: [T, ld] activations, a row holding q [H, D] | k [H, D] | v [H, E] | z [H, E];
// gates: float [T, 2H] (input gates, then forget gates, before bias and cap); out: [T, H * E].
static int mlstm_run(bool direct, const void* qkvz, int ld, const float* gates, const float* bias_i, const float* bias_f,
                     const float* norm_w, float* state, int slot_words, int offset_words, const int* q_start,
                     const int* slot_of_req, void* out, int R, int H, int D, int E, float cap, float eps, void* stream) {
  ZK_REQUIRE(R >= 0 && H > 0 && H <= 65535 && D > 0 && E > 0, "zk_mlstm: bad sizes");
  ZK_REQUIRE(E <= MLSTM_THREADS, "zk_mlstm: more than 256 value channels a head are not supported");
  ZK_REQUIRE(ld >= 2 * H * (D + E), "zk_mlstm: rows too short");
  ZK_REQUIRE(cap > 0.f, "zk_mlstm: the gates' cap must be positive");
  ZK_REQUIRE((size_t)slot_words * 4 >= (size_t)offset_words * 4 + zk_mlstm_state_bytes(H, D, E),
             "zk_mlstm: the state does not fit its slot");
  if (R == 0) return 0;
  // a head's S that does not fit the local memory stays in the state slot (the same bits, slower)
  if (!direct && ((size_t)D * E + 3 * D + E + MLSTM_THREADS + 32) * 4 > 150 * 1024) direct = true;
  const size_t lds = ((direct ? 0 : (size_t)D * E) + 3 * D + E + MLSTM_THREADS + 32) * 4;
  ZK_REQUIRE(lds <= 160 * 1024, "zk_mlstm: a head's state does not fit the local memory");
  if (lds > 48 * 1024) {
    static size_t raised = 0;
    if (lds > raised) {
      hipFuncSetAttribute((const void*)mlstm_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      raised = lds;
    }
  }
  dim3 grid(R, H);
  if (direct)
    mlstm_kernel<true><<<grid, MLSTM_THREADS, lds, (hipStream_t)stream>>>(
        (const act_t*)qkvz, ld, gates, bias_i, bias_f, norm_w, state, slot_words, offset_words, q_start, slot_of_req,
        (act_t*)out, H, D, E, cap, eps, 1.0f / sqrtf((float)D));
  else
    mlstm_kernel<false><<<grid, MLSTM_THREADS, lds, (hipStream_t)stream>>>(
        (const act_t*)qkvz, ld, gates, bias_i, bias_f, norm_w, state, slot_words, offset_words, q_start, slot_of_req,
        (act_t*)out, H, D, E, cap, eps, 1.0f / sqrtf((float)D));
  return zk_launch_status("zk_mlstm");
}

int zk_mlstm(const void* qkvz, int ld, const float* gates, const float* bias_i, const float* bias_f,
             const float* norm_w, float* state, int slot_words, int offset_words, const int* q_start,
             const int* slot_of_req, void* out, int R, int H, int D, int E, float cap, float eps, void* stream) {
  return mlstm_run(false, qkvz, ld, gates, bias_i, bias_f, norm_w, state, slot_words, offset_words, q_start, slot_of_req,
                   out, R, H, D, E, cap, eps, stream);
}

// The same for steps in which every request brings one token: the state is renewed where it lies.
// (Right for any step, and bit for bit what zk_mlstm gives; only slower where requests bring more.)
int zk_mlstm_token(const void* qkvz, int ld, const float* gates, const float* bias_i, const float* bias_f,
                   const float* norm_w, float* state, int slot_words, int offset_words, const int* q_start,
                   const int* slot_of_req, void* out, int R, int H, int D, int E, float cap, float eps, void* stream) {
  return mlstm_run(true, qkvz, ld, gates, bias_i, bias_f, norm_w, state, slot_words, offset_words, q_start, slot_of_req,
                   out, R, H, D, E, cap, eps, stream);
}

// The same as zk_mlstm for steps that bring portions: chunks of up to 64 tokens (fewer where
// max_q_len, the longest portion of the step, or the local memory asks for less).  o_raw: float
// [T, H * E] scratch; nm_new: float [R, H, D + 1] scratch.  zk_mlstm_finish must follow.
int zk_mlstm_chunked(const void* qkvz, int ld, const float* gates, const float* bias_i, const float* bias_f,
                     float* state, int slot_words, int offset_words, const int* q_start, const int* slot_of_req,
                     float* o_raw, float* nm_new, int R, int H, int D, int E, float cap, int max_q_len, void* stream) {
  ZK_REQUIRE(R >= 0 && R <= 65535 && H > 0 && H <= 65535 && D > 0 && E > 0, "zk_mlstm_chunked: bad sizes");
  ZK_REQUIRE(D <= 256 && E <= 2048, "zk_mlstm_chunked: heads of more than 256 key channels are not supported");
  ZK_REQUIRE(ld >= 2 * H * (D + E), "zk_mlstm_chunked: rows too short");
  ZK_REQUIRE(cap > 0.f, "zk_mlstm_chunked: the gates' cap must be positive");
  ZK_REQUIRE((size_t)slot_words * 4 >= (size_t)offset_words * 4 + zk_mlstm_state_bytes(H, D, E),
             "zk_mlstm_chunked: the state does not fit its slot");
  if (R == 0) return 0;
  int L = max_q_len <= 16 ? 16 : max_q_len <= 32 ? 32 : 64;
  while (L > 16 && mlstm_chunk_lds(L, D) > 150 * 1024) L /= 2;
  hipStream_t s = (hipStream_t)stream;
#define ZK_CHUNK_(L_) \
  mlstm_chunk_launch<L_>(qkvz, ld, gates, bias_i, bias_f, state, slot_words, offset_words, q_start, slot_of_req, o_raw, \
                         nm_new, R, H, D, E, cap, s)
  return L == 64 ? ZK_CHUNK_(64) : L == 32 ? ZK_CHUNK_(32) : ZK_CHUNK_(16);
#undef ZK_CHUNK_
}

}  // extern "C"

static int mlstm_scan_len(int max_q_len, int D) {
  int L = max_q_len <= 16 ? 16 : max_q_len <= 32 ? 32 : 64;
  while (L > 16 && mlstm_chunk_lds(L, D) > 150 * 1024) L /= 2;
  return L;
}

// Floats of scratch that zk_mlstm_scan needs for a step of T tokens in R requests.
extern "C" size_t zk_mlstm_scan_floats(int T, int R, int H, int D, int E, int max_q_len) {
  const int L = mlstm_scan_len(max_q_len, D);
  const size_t chunks = (size_t)(T + L - 1) / L + R;
  return chunks * H * ((size_t)D * E + D + 3);
}

template <int L>
static int mlstm_scan_launch(const void* qkvz, int ld, const float* gates, const float* bias_i, const float* bias_f,
                             float* state, int slot_words, int offset_words, const int* q_start, const int* slot_of_req,
                             float* o_raw, float* work, int chunks, int R, int H, int D, int E, float cap, hipStream_t s) {
  float* Uw = work;
  float* uw = Uw + (size_t)chunks * H * D * E;
  float* af = uw + (size_t)chunks * H * D;
  float* mprev = af + (size_t)chunks * H * 2;
  const int zs = (E + MLSTM_EC - 1) / MLSTM_EC;
  const size_t lds_local = ((size_t)L * (D + 1) + (size_t)L * MLSTM_EC + 3 * L + 8) * 4;
  const size_t lds_out = mlstm_chunk_lds(L, D);
  static size_t raised_local = 0, raised_out = 0;
  if (lds_local > 48 * 1024 && lds_local > raised_local) {
    hipFuncSetAttribute((const void*)mlstm_local_kernel<L>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_local);
    raised_local = lds_local;
  }
  if (lds_out > 48 * 1024 && lds_out > raised_out) {
    hipFuncSetAttribute((const void*)mlstm_output_kernel<L>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_out);
    raised_out = lds_out;
  }
  mlstm_local_kernel<L><<<dim3(chunks, H, zs), MLSTM_THREADS, lds_local, s>>>((const act_t*)qkvz, ld, gates, bias_i, bias_f,
                                                                              q_start, Uw, uw, af, R, H, D, E, cap);
  if (int rc = zk_launch_status("zk_mlstm_scan (local)")) return rc;
  mlstm_scan_kernel<<<dim3(R, H, (D * E + D + 1 + MLSTM_THREADS - 1) / MLSTM_THREADS), MLSTM_THREADS, 0, s>>>(
      state, slot_words, offset_words, q_start, slot_of_req, Uw, uw, af, mprev, L, H, D, E);
  if (int rc = zk_launch_status("zk_mlstm_scan (scan)")) return rc;
  mlstm_output_kernel<L><<<dim3(chunks, H, zs), MLSTM_THREADS, lds_out, s>>>((const act_t*)qkvz, ld, gates, bias_i, bias_f,
                                                                             q_start, Uw, uw, mprev, o_raw, R, H, D, E, cap,
                                                                             1.0f / sqrtf((float)D));
  return zk_launch_status("zk_mlstm_scan (output)");
}

extern "C" {

// zk_mlstm_chunked's work with the chunks of a step side by side (three launches); for steps
// whose portions are several chunks long.  work: zk_mlstm_scan_floats(...) floats of scratch.
// zk_mlstm_finish (with nm_new null: the scan stores n and m itself) must follow.
int zk_mlstm_scan(const void* qkvz, int ld, const float* gates, const float* bias_i, const float* bias_f, float* state,
                  int slot_words, int offset_words, const int* q_start, const int* slot_of_req, float* o_raw, float* work,
                  size_t work_floats, int T, int R, int H, int D, int E, float cap, int max_q_len, void* stream) {
  ZK_REQUIRE(T >= 0 && R >= 0 && R <= 65535 && H > 0 && H <= 65535 && D > 0 && E > 0, "zk_mlstm_scan: bad sizes");
  ZK_REQUIRE(D <= 256 && E <= 2048, "zk_mlstm_scan: heads of more than 256 key channels are not supported");
  ZK_REQUIRE(ld >= 2 * H * (D + E), "zk_mlstm_scan: rows too short");
  ZK_REQUIRE(cap > 0.f, "zk_mlstm_scan: the gates' cap must be positive");
  ZK_REQUIRE((size_t)slot_words * 4 >= (size_t)offset_words * 4 + zk_mlstm_state_bytes(H, D, E),
             "zk_mlstm_scan: the state does not fit its slot");
  ZK_REQUIRE(work != nullptr && work_floats >= zk_mlstm_scan_floats(T, R, H, D, E, max_q_len), "zk_mlstm_scan: too little scratch");
  if (R == 0 || T == 0) return 0;
  const int L = mlstm_scan_len(max_q_len, D);
  const int chunks = (T + L - 1) / L + R;
  hipStream_t s = (hipStream_t)stream;
#define ZK_SCAN_(L_) \
  mlstm_scan_launch<L_>(qkvz, ld, gates, bias_i, bias_f, state, slot_words, offset_words, q_start, slot_of_req, o_raw, work, \
                        chunks, R, H, D, E, cap, s)
  return L == 64 ? ZK_SCAN_(64) : L == 32 ? ZK_SCAN_(32) : ZK_SCAN_(16);
#undef ZK_SCAN_
}

int zk_mlstm_finish(const float* o_raw, const void* qkvz, int ld, const float* norm_w, const float* nm_new,
                    float* state, int slot_words, int offset_words, const int* req_of_token, const int* q_start,
                    const int* slot_of_req, void* out, int T, int H, int D, int E, float eps, void* stream) {
  ZK_REQUIRE(T >= 0 && H > 0 && H <= 65535 && D > 0 && E > 0, "zk_mlstm_finish: bad sizes");
  if (T == 0) return 0;
  dim3 grid(T, H);
  mlstm_finish_kernel<<<grid, 64, 0, (hipStream_t)stream>>>(o_raw, (const act_t*)qkvz, ld, norm_w, nm_new, state,
                                                            slot_words, offset_words, req_of_token, q_start, slot_of_req,
                                                            (act_t*)out, H, D, E, eps);
  return zk_launch_status("zk_mlstm_finish");
}

}  // extern "C"

ZK_ENTER(zk_mlstm)
ZK_ENTER(zk_mlstm_token)
ZK_ENTER(zk_mlstm_chunked)
ZK_ENTER(zk_mlstm_scan)
ZK_ENTER(zk_mlstm_finish)
