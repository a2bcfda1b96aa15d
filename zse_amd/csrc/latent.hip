// Attention over one latent row per token.
//
// A token leaves c = rms_norm(first C channels of its down-projection) * gain and one rotated key
// part of R channels; head h's key would be [Wuk_h c, rotated part] and its value Wuv_h c.  Only
// [c, rotated part] is cached (one "key head" of C + R channels).  Because
//     q_plain . (Wuk_h c) = (Wuk_h^T q_plain) . c      and      sum_j p_j (Wuv_h c_j) = Wuv_h (sum_j p_j c_j)
// a query head becomes [Wuk_h^T q_plain, q_rotated] (C + R channels), attends to the cached rows
// as keys and to their first C channels as values, and the result goes through Wuv_h.  The two
// per-head products are ``zk_heads_linear``; ``zk_latent_prep`` norms, rotates and stores.
#include "common.h"
#include "packed_call.h"

extern "C" int zk_steplist_register(const char* name, int nargs, void* fn);
#define ZK_ENTER(fn) \
  static const int fn##_entered = zk_steplist_register(#fn, zk_packed::Call<fn>::nargs, (void*)zk_packed::Call<fn>::call);

// One block per (token, head or latent).  Heads: the rotated part of the query goes, rotated, to
// qa[t, head, C:].  The latent (blockIdx.y == H): the normed c and the rotated key part go to
// the cache row of the token's slot.
__global__ __launch_bounds__(256) void latent_prep_kernel(
    const act_t* __restrict__ qd, int ld, const int* __restrict__ positions, const int* __restrict__ slot_map,
    const float* __restrict__ gain, float eps, const float* __restrict__ freq, float rot_scale, int interleaved,
    act_t* __restrict__ qa, act_t* __restrict__ kcache, int H, int D, int R, int C, int bs) {
  __shared__ float red[17];
  const int t = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
  const int pos = positions[t];
  if (pos < 0) return;
  const int half = R / 2;
  if (head < H) {
    const act_t* src = qd + (size_t)t * ld + (size_t)head * (D + R) + D;
    act_t* dst = qa + ((size_t)t * H + head) * (C + R) + C;
    for (int m = tid; m < half; m += 256) {
      float sn, cs, ra, rb;
      sincosf((float)pos * freq[m], &sn, &cs);
      sn *= rot_scale;
      cs *= rot_scale;
      const int ia = interleaved ? 2 * m : m, ib = interleaved ? 2 * m + 1 : m + half;
      rotate_pair(to_f32(src[ia]), to_f32(src[ib]), sn, cs, ra, rb);
      dst[ia] = from_f32<act_t>(ra);
      dst[ib] = from_f32<act_t>(rb);
    }
    return;
  }
  const int slot = slot_map[t];
  if (slot < 0) return;
  const act_t* src = qd + (size_t)t * ld + (size_t)H * (D + R);
  act_t* dst = kcache + (size_t)slot * (C + R);           // one key head: row (page * bs + offset)
  float ss = 0.f;
  for (int i = tid; i < C; i += 256) {
    const float x = to_f32(src[i]);
    ss = fmaf(x, x, ss);
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)C + eps);
  for (int i = tid; i < C; i += 256) dst[i] = from_f32<act_t>(to_f32(src[i]) * inv * gain[i]);
  for (int m = tid; m < half; m += 256) {
    float sn, cs, ra, rb;
    sincosf((float)pos * freq[m], &sn, &cs);
    sn *= rot_scale;
    cs *= rot_scale;
    const int ia = interleaved ? 2 * m : m, ib = interleaved ? 2 * m + 1 : m + half;
    rotate_pair(to_f32(src[C + ia]), to_f32(src[C + ib]), sn, cs, ra, rb);
    dst[C + ia] = from_f32<act_t>(ra);
    dst[C + ib] = from_f32<act_t>(rb);
  }
}

// out[t, h, n] = sum_k x[t, h, k] w_h(n, k);  w_h(n, k) = w[(h K + k) N + n] (kn) or w[(h N + n) K + k].
// A block: 32 tokens x 64 columns of one head; a thread: 8 tokens of one column.
#define HL_TT 32
#define HL_TK 32
template <bool KN>
__global__ __launch_bounds__(256) void heads_linear_kernel(const act_t* __restrict__ x, int ldx, int x_head,
                                                           const act_t* __restrict__ w, act_t* __restrict__ out, int ldo,
                                                           int o_head, int T, int K, int N) {
  __shared__ float xs[HL_TT][HL_TK + 1];
  __shared__ float ws[HL_TK][64 + 1];
  const int h = blockIdx.y, t0 = blockIdx.x * HL_TT, n0 = blockIdx.z * 64;
  const int tid = threadIdx.x, tx = tid & 63, ty = tid >> 6;
  const act_t* wh = w + (size_t)h * K * N;
  float acc[8] = {};
  for (int k0 = 0; k0 < K; k0 += HL_TK) {
    __syncthreads();
    for (int i = tid; i < HL_TT * HL_TK; i += 256) {
      const int tt = i / HL_TK, kk = i % HL_TK;
      xs[tt][kk] = (t0 + tt < T && k0 + kk < K) ? to_f32(x[(size_t)(t0 + tt) * ldx + (size_t)h * x_head + k0 + kk]) : 0.f;
    }
    for (int i = tid; i < HL_TK * 64; i += 256) {
      int kk, nn;
      if (KN) {
        kk = i / 64;
        nn = i % 64;
      } else {
        nn = i / HL_TK;
        kk = i % HL_TK;
      }
      const bool in = k0 + kk < K && n0 + nn < N;
      ws[kk][nn] = in ? to_f32(KN ? wh[(size_t)(k0 + kk) * N + n0 + nn] : wh[(size_t)(n0 + nn) * K + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < HL_TK; kk++) {
      const float wv = ws[kk][tx];
#pragma unroll
      for (int j = 0; j < 8; j++) acc[j] = fmaf(xs[ty * 8 + j][kk], wv, acc[j]);
    }
  }
  if (n0 + tx < N) {
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const int t = t0 + ty * 8 + j;
      if (t < T) out[(size_t)t * ldo + (size_t)h * o_head + n0 + tx] = from_f32<act_t>(acc[j]);
    }
  }
}

extern "C" {

// qd: [T, ld]: H query heads of D + R, then C + R of the down-projection.  qa: [T, H, C + R], of
// which this writes [.., C:].  kcache: [pages, 1, bs, C + R].  freq: float [R / 2].
int zk_latent_prep(const void* qd, int ld, const int* positions, const int* slot_map, const float* gain, float eps,
                   const float* freq, float rot_scale, int interleaved, void* qa, void* kcache, int T, int H, int D,
                   int R, int C, int bs, void* stream) {
  ZK_REQUIRE(T >= 0 && H > 0 && D > 0 && R >= 0 && R % 2 == 0 && C > 0 && bs > 0, "zk_latent_prep: bad sizes");
  ZK_REQUIRE(ld >= H * (D + R) + C + R, "zk_latent_prep: rows too short");
  ZK_REQUIRE(H < 65535 && (R == 0 || freq != nullptr), "zk_latent_prep: too many heads, or no frequencies");
  if (T == 0) return 0;
  dim3 grid(T, H + 1);
  latent_prep_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const act_t*)qd, ld, positions, slot_map, gain, eps, freq,
                                                            rot_scale, interleaved, (act_t*)qa, (act_t*)kcache, H, D, R, C, bs);
  return zk_launch_status("zk_latent_prep");
}

// x: head h of token t at x[t * ldx + h * x_head], K channels; out likewise with ldo, o_head, N.
// w: [H][K][N] when w_kn, else [H][N][K].
int zk_heads_linear(const void* x, int ldx, int x_head, const void* w, int w_kn, void* out, int ldo, int o_head, int T,
                    int H, int K, int N, void* stream) {
  ZK_REQUIRE(T >= 0 && H > 0 && K > 0 && N > 0, "zk_heads_linear: bad sizes");
  ZK_REQUIRE(H <= 65535 && (N + 63) / 64 <= 65535, "zk_heads_linear: too many heads or columns");
  if (T == 0) return 0;
  dim3 grid((T + HL_TT - 1) / HL_TT, H, (N + 63) / 64);
  if (w_kn)
    heads_linear_kernel<true><<<grid, 256, 0, (hipStream_t)stream>>>((const act_t*)x, ldx, x_head, (const act_t*)w,
                                                                     (act_t*)out, ldo, o_head, T, K, N);
  else
    heads_linear_kernel<false><<<grid, 256, 0, (hipStream_t)stream>>>((const act_t*)x, ldx, x_head, (const act_t*)w,
                                                                      (act_t*)out, ldo, o_head, T, K, N);
  return zk_launch_status("zk_heads_linear");
}

}  // extern "C"

ZK_ENTER(zk_latent_prep)
ZK_ENTER(zk_heads_linear)
