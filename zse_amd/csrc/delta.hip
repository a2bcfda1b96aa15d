// The gated delta rule: a recurrent mixer with a matrix state S [D, E] per head.
//
//   S <- g_t S;   u_t = beta_t (v_t - S^T k_t);   S <- S + k_t u_t^T;   o_t = S^T q_t
//
// with q_t, k_t made unit vectors per head (x / sqrt(sum x^2 + 1e-6), q also times D^(-1/2)),
// beta_t = sigmoid(b_t), g_t = exp(-exp(A) softplus(a_t + dt)), and the read-out divided by its
// root mean square over E, times a gain [E] and silu(z_t).
//
// The recurrence never mixes value channels: column e of S, u and o depend on column e alone.
// So a thread owns one column of S, D floats in registers, and walks the tokens of its request
// without talking to any other thread; q_t and k_t are read from local memory by every thread
// at the same address (a broadcast).  Tokens are staged in groups: the block loads and
// normalises q and k of a group, walks it, then norms and gates the group's read-outs.  Every
// sum runs in an order fixed by the channel numbers alone, so a request's values are the same
// bits however its tokens are cut into steps.  All arithmetic is float; q, k, v, z come in the
// activation type, b and a as floats.
#include "common.h"
#include "packed_call.h"

extern "C" int zk_steplist_register(const char* name, int nargs, void* fn);
#define ZK_ENTER(fn) \
  static const int fn##_entered = zk_steplist_register(#fn, zk_packed::Call<fn>::nargs, (void*)zk_packed::Call<fn>::call);

#define DELTA_GROUP 16

__device__ __forceinline__ float softplus_f(float x) {
  // log(1 + exp(x)) without overflow
  return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
}

template <int DMAX>
__global__ void delta_rule_kernel(const act_t* __restrict__ qkv, int ld, int k_off, int v_off,
                                  const act_t* __restrict__ z, int ldz, const float* __restrict__ ba,
                                  const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                                  const float* __restrict__ gain, float* __restrict__ state, int slot_words,
                                  int offset_words, const int* __restrict__ q_start,
                                  const int* __restrict__ slot_of_req, act_t* __restrict__ out, int H, int G, int D,
                                  int E, int Epad, float eps) {
  extern __shared__ float lds[];
  float* qs = lds;                                 // [GROUP][DMAX]
  float* ks = qs + DELTA_GROUP * DMAX;             // [GROUP][DMAX]
  float* ov = ks + DELTA_GROUP * DMAX;             // [GROUP][Epad]: v going in, the read-out coming back
  float* beta = ov + DELTA_GROUP * Epad;           // [GROUP]
  float* dec = beta + DELTA_GROUP;                 // [GROUP]
  const int r = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, nt = blockDim.x;
  const int lane = tid & 63, wave = tid >> 6, nw = nt >> 6;
  const int t0 = q_start[r], t1 = q_start[r + 1];
  if (t1 <= t0) return;
  const int g = h / (H / G);
  const bool live = tid < E;
  float* S = state + (size_t)slot_of_req[r] * slot_words + offset_words + (size_t)h * D * E;
  float s[DMAX];
#pragma unroll
  for (int d = 0; d < DMAX; d++) s[d] = (live && d < D) ? S[(size_t)d * E + tid] : 0.f;
  const float rate = expf(A_log[h]), shift = dt_bias[h];
  const float q_scale = 1.0f / sqrtf((float)D);
  for (int c0 = t0; c0 < t1; c0 += DELTA_GROUP) {
    const int n = min(DELTA_GROUP, t1 - c0);
    __syncthreads();
    for (int i = tid; i < n * DMAX; i += nt) {
      const int tt = i / DMAX, d = i % DMAX;
      const act_t* row = qkv + (size_t)(c0 + tt) * ld + (size_t)g * D;
      qs[i] = d < D ? to_f32(row[d]) : 0.f;
      ks[i] = d < D ? to_f32(row[k_off + d]) : 0.f;
    }
    for (int i = tid; i < n * Epad; i += nt) {
      const int tt = i / Epad, e = i % Epad;
      ov[i] = e < E ? to_f32(qkv[(size_t)(c0 + tt) * ld + v_off + (size_t)h * E + e]) : 0.f;
    }
    if (tid < n) {
      const float* row = ba + (size_t)(c0 + tid) * 2 * H;
      beta[tid] = 1.0f / (1.0f + expf(-row[h]));
      dec[tid] = expf(-rate * softplus_f(row[H + h] + shift));
    }
    __syncthreads();
    for (int tt = wave; tt < n; tt += nw) {        // unit vectors
      float sq = 0.f, sk = 0.f;
      for (int d = lane; d < DMAX; d += 64) {
        sq = fmaf(qs[tt * DMAX + d], qs[tt * DMAX + d], sq);
        sk = fmaf(ks[tt * DMAX + d], ks[tt * DMAX + d], sk);
      }
      sq = wave_sum(sq);
      sk = wave_sum(sk);
      const float iq = q_scale / sqrtf(sq + 1e-6f), ik = 1.0f / sqrtf(sk + 1e-6f);
      for (int d = lane; d < DMAX; d += 64) {
        qs[tt * DMAX + d] *= iq;
        ks[tt * DMAX + d] *= ik;
      }
    }
    __syncthreads();
    for (int tt = 0; tt < n; tt++) {               // the walk: nothing is shared between threads
      const float4* k4 = (const float4*)(ks + tt * DMAX);
      const float4* q4 = (const float4*)(qs + tt * DMAX);
      const float gt = dec[tt];
      float dot = 0.f;
#pragma unroll
      for (int d = 0; d < DMAX / 4; d++) {
        const float4 kk = k4[d];
        s[4 * d] *= gt;
        s[4 * d + 1] *= gt;
        s[4 * d + 2] *= gt;
        s[4 * d + 3] *= gt;
        dot = fmaf(s[4 * d], kk.x, dot);
        dot = fmaf(s[4 * d + 1], kk.y, dot);
        dot = fmaf(s[4 * d + 2], kk.z, dot);
        dot = fmaf(s[4 * d + 3], kk.w, dot);
      }
      const float u = beta[tt] * (ov[tt * Epad + (live ? tid : 0)] - dot);
      float o = 0.f;
#pragma unroll
      for (int d = 0; d < DMAX / 4; d++) {
        const float4 kk = k4[d], qq = q4[d];
        s[4 * d] = fmaf(kk.x, u, s[4 * d]);
        s[4 * d + 1] = fmaf(kk.y, u, s[4 * d + 1]);
        s[4 * d + 2] = fmaf(kk.z, u, s[4 * d + 2]);
        s[4 * d + 3] = fmaf(kk.w, u, s[4 * d + 3]);
        o = fmaf(s[4 * d], qq.x, o);
        o = fmaf(s[4 * d + 1], qq.y, o);
        o = fmaf(s[4 * d + 2], qq.z, o);
        o = fmaf(s[4 * d + 3], qq.w, o);
      }
      if (live) ov[tt * Epad + tid] = o;
    }
    __syncthreads();
    for (int tt = wave; tt < n; tt += nw) {        // unit RMS over the head's read-out, gain, gate
      float ss = 0.f;
      for (int e = lane; e < E; e += 64) ss = fmaf(ov[tt * Epad + e], ov[tt * Epad + e], ss);
      ss = wave_sum(ss);
      const float inv = 1.0f / sqrtf(ss / (float)E + eps);
      const act_t* zr = z + (size_t)(c0 + tt) * ldz + (size_t)h * E;
      act_t* orow = out + ((size_t)(c0 + tt) * H + h) * E;
      for (int e = lane; e < E; e += 64) {
        const float zz = to_f32(zr[e]);
        orow[e] = from_f32<act_t>(ov[tt * Epad + e] * inv * gain[e] * (zz / (1.0f + expf(-zz))));
      }
    }
  }
  if (live) {
#pragma unroll
    for (int d = 0; d < DMAX; d++)
      if (d < D) S[(size_t)d * E + tid] = s[d];
  }
}

extern "C" {

// qkv: [T, ld] activations after the convolution and silu: G query heads of D at column 0, G key
// heads at k_off, H value heads of E at v_off.  z: [T, ldz], H heads of E (the output gate before
// its silu).  ba: float [T, 2H], b then a.  A_log, dt_bias: float [H]; gain: float [E].
// state: request r's S [H, D, E] lies at state[slot_of_req[r] * slot_words + offset_words].
// out: [T, H * E].  Requests are rows [q_start[r], q_start[r + 1]).
int zk_delta_rule(const void* qkv, int ld, int k_off, int v_off, const void* z, int ldz, const float* ba,
                  const float* A_log, const float* dt_bias, const float* gain, float* state, int slot_words,
                  int offset_words, const int* q_start, const int* slot_of_req, void* out, int R, int H, int G, int D,
                  int E, float eps, void* stream) {
  ZK_REQUIRE(R >= 0 && H > 0 && G > 0 && H % G == 0 && D > 0 && E > 0, "zk_delta_rule: bad sizes");
  ZK_REQUIRE(D <= 256, "zk_delta_rule: up to 256 query/key channels a head");
  ZK_REQUIRE(E <= 1024, "zk_delta_rule: up to 1024 value channels a head");
  ZK_REQUIRE(H <= 65535, "zk_delta_rule: too many heads");
  ZK_REQUIRE(state != nullptr && slot_words >= offset_words + H * D * E, "zk_delta_rule: the state does not fit its slot");
  if (R == 0) return 0;
  const int threads = (E + 63) / 64 * 64, Epad = threads;
  const int DMAX = D <= 32 ? 32 : D <= 64 ? 64 : D <= 128 ? 128 : 256;
  const size_t lds = ((size_t)DELTA_GROUP * (2 * DMAX + Epad) + 2 * DELTA_GROUP) * sizeof(float);
  dim3 grid(R, H);
#define LAUNCH(N)                                                                                                      \
  do {                                                                                                                 \
    static bool raised = false;                                                                                        \
    if (lds > 48 * 1024 && !raised) {                                                                                  \
      hipFuncSetAttribute((const void*)delta_rule_kernel<N>, hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024); \
      raised = true;                                                                                                   \
    }                                                                                                                  \
    delta_rule_kernel<N><<<grid, threads, lds, (hipStream_t)stream>>>(                                                 \
        (const act_t*)qkv, ld, k_off, v_off, (const act_t*)z, ldz, ba, A_log, dt_bias, gain, state, slot_words,        \
        offset_words, q_start, slot_of_req, (act_t*)out, H, G, D, E, Epad, eps);                                       \
  } while (0)
  if (DMAX == 32) LAUNCH(32);
  else if (DMAX == 64) LAUNCH(64);
  else if (DMAX == 128) LAUNCH(128);
  else LAUNCH(256);
#undef LAUNCH
  return zk_launch_status("zk_delta_rule");
}

}  // extern "C"

ZK_ENTER(zk_delta_rule)
