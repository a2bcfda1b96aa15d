// The gated delta rule: a recurrent mixer with a matrix state S [D, E] per head.
//
//   S <- g_t S;   u_t = beta_t (v_t - S^T k_t);   S <- S + k_t u_t^T;   o_t = S^T q_t
//
// with q_t, k_t made unit vectors per head (x / sqrt(sum x^2 + 1e-6), q also times D^(-1/2)),
// beta_t = sigmoid(b_t), g_t = exp(-exp(A) softplus(a_t + dt)), and the read-out divided by its
// root mean square over E, times a gain [E] and silu(z_t).
//
// The recurrence never mixes value channels: column e of S, u and o depend on column e alone.
// Eight neighbouring lanes own one column of S, each a share of its rows in registers (row
// chunks of four, dealt out in turn), and walk the tokens of their request; the two sums over
// the rows (S^T k and S^T q) are joined across the eight lanes by three lane permutations inside
// the wave, no local memory and no barrier.  q_t and k_t are read from local memory, every
// column at the same addresses.  Tokens are staged in groups: the block loads and normalises q
// and k of a group, walks it, then norms and gates the group's read-outs (a head whose value
// channels span several blocks leaves that to a second kernel).  Every sum runs in an order
// fixed by the channel numbers alone, so a request's values are the same bits however its
// tokens are cut into steps.  All arithmetic is float; q, k, v, z come in the activation type,
// b and a as floats.
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

// Eight consecutive activations as they lie in memory (16 bytes of bfloat16, or 32 of float, a
// lane), turned into floats only when they are put down in local memory.
#if ZSE_ACT_BF16
typedef __bf16 Eight __attribute__((ext_vector_type(8)));
__device__ __forceinline__ Eight load8(const __bf16* p) { return *(const Eight*)p; }
__device__ __forceinline__ float at8(const Eight& e, int i) { return (float)e[i]; }
#else
struct Eight {
  float4 a, b;
};
__device__ __forceinline__ Eight load8(const float* p) { return Eight{*(const float4*)p, *(const float4*)(p + 4)}; }
__device__ __forceinline__ float at8(const Eight& e, int i) {
  const float4 h = i < 4 ? e.a : e.b;
  const int c = i & 3;
  return c == 0 ? h.x : c == 1 ? h.y : c == 2 ? h.z : h.w;
}
#endif

#define DELTA_COLS 128            // the most value channels a block takes (8 lanes each: 1024 threads)
#define DELTA_COLS_LONG 16        // and what it takes when portions are long: 16 lanes a column, more blocks, one wave a SIMD

// The sum of x over the 8 lanes that share a column: lane i with 7 - i, then inside the quads.
__device__ __forceinline__ float sum8(float x) {
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x141, 0xf, 0xf, false));   // row_half_mirror
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0xB1, 0xf, 0xf, false));    // quad_perm [1,0,3,2]
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x4E, 0xf, 0xf, false));    // quad_perm [2,3,0,1]
  return x;
}

// The sum over the 16 lanes of a row that share a column: lane i with 15 - i first.
__device__ __forceinline__ float sum16(float x) {
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x140, 0xf, 0xf, false));   // row_mirror
  return sum8(x);
}

// DS lanes share a column (8 or 16), each holds CH chunks of four rows of S (4 CH DS rows in all,
// D padded with zeros).  raw (may be null): float [T, H * E], the read-outs before their norm,
// for a head that spans several blocks.  GRP: tokens staged at a time.  PRE: pieces of eight q/k
// values a thread carries for the next group of tokens (4: blocks of up to 256 threads, for long
// portions; 1: blocks of up to 1024).
template <int CH, int DS, int PRE>
__global__ __launch_bounds__(PRE > 1 ? 256 : 1024) void delta_rule_kernel(
    const act_t* __restrict__ qkv, int ld, int k_off, int v_off, const act_t* __restrict__ z, int ldz,
    const float* __restrict__ ba, const float* __restrict__ A_log, const float* __restrict__ dt_bias,
    const float* __restrict__ gain, float* __restrict__ state, int slot_words, int offset_words,
    const int* __restrict__ q_start, const int* __restrict__ slot_of_req, act_t* __restrict__ out,
    float* __restrict__ raw, int H, int G, int D, int E, float eps, int COLS, int GRP, int wide) {
  constexpr int DMAX = 4 * CH * DS, RD = 4 * CH;     // RD: rows of S a lane holds; COLS: value channels of this block
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* qs = lds;                                 // [GRP][DMAX]
  float* ks = qs + GRP * DMAX;                     // [GRP][DMAX]
  float* ov = ks + GRP * DMAX;                     // [GRP][COLS]: v going in, the read-out coming back
  float* beta = ov + GRP * COLS;                   // [GRP]
  float* dec = beta + GRP;                         // [GRP]
  const int r = blockIdx.x, h = blockIdx.y, e0 = blockIdx.z * COLS, tid = threadIdx.x, nt = blockDim.x;
  const int lane = tid & 63, wave = tid >> 6, nw = nt >> 6;
  const int col = tid / DS, j = tid % DS, e = e0 + col;
  const int t0 = q_start[r], t1 = q_start[r + 1];
  if (t1 <= t0) return;
  const int g = h / (H / G);
  const bool live = e < E;
  const int cols = min(COLS, E - e0);
  float* S = state + (size_t)slot_of_req[r] * slot_words + offset_words + (size_t)h * D * E;
  float s[RD];
#pragma unroll
  for (int i = 0; i < CH; i++)
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const int d = 4 * (j + DS * i) + c;
      s[4 * i + c] = (live && d < D) ? S[(size_t)d * E + e] : 0.f;
    }
  const float rate = expf(A_log[h]), shift = dt_bias[h];
  const float q_scale = 1.0f / sqrtf((float)D);
  // wide: rows in whole groups of eight values.  A group's q, k, v, b and a are then asked for, 16
  // bytes a lane, while the group before it is walked, and land in local memory afterwards.
  const int qk_pieces = D / 8;                       // of one row of q (or k)
  Eight pq[PRE], pv;
  float pb = 0.f, pa = 0.f;
  auto fetch = [&](int c0, int n) {
#pragma unroll
    for (int u = 0; u < PRE; u++) {
      const int i = tid + u * nt;
      if (i < 2 * n * qk_pieces) {
        const int which = i / (n * qk_pieces), rest = i % (n * qk_pieces);
        const int tt = rest / qk_pieces, d8 = (rest % qk_pieces) * 8;
        pq[u] = load8(qkv + (size_t)(c0 + tt) * ld + (size_t)g * D + (which ? k_off : 0) + d8);
      }
    }
    if (tid < n * (COLS / 8)) {
      const int tt = tid / (COLS / 8), c8 = (tid % (COLS / 8)) * 8;
      if (c8 < cols) pv = load8(qkv + (size_t)(c0 + tt) * ld + v_off + (size_t)h * E + e0 + c8);
    }
    if (tid < n) {
      const float* row = ba + (size_t)(c0 + tid) * 2 * H;
      pb = row[h];
      pa = row[H + h];
    }
  };
  if (wide) {
    for (int i = tid; i < GRP * DMAX; i += nt) qs[i] = ks[i] = 0.f;       // the rows' padding stays zero
    for (int i = tid; i < GRP * COLS; i += nt) ov[i] = 0.f;
    fetch(t0, min(GRP, t1 - t0));
  }
  for (int c0 = t0; c0 < t1; c0 += GRP) {
    const int n = min(GRP, t1 - c0);
    __syncthreads();
    if (wide) {
#pragma unroll
      for (int u = 0; u < PRE; u++) {
        const int i = tid + u * nt;
        if (i < 2 * n * qk_pieces) {
          const int which = i / (n * qk_pieces), rest = i % (n * qk_pieces);
          const int tt = rest / qk_pieces, d8 = (rest % qk_pieces) * 8;
          float* dst = (which ? ks : qs) + tt * DMAX + d8;
#pragma unroll
          for (int c = 0; c < 8; c++) dst[c] = at8(pq[u], c);
        }
      }
      if (tid < n * (COLS / 8)) {
        const int tt = tid / (COLS / 8), c8 = (tid % (COLS / 8)) * 8;
        if (c8 < cols) {
#pragma unroll
          for (int c = 0; c < 8; c++) ov[tt * COLS + c8 + c] = at8(pv, c);
        }
      }
      if (tid < n) {
        beta[tid] = 1.0f / (1.0f + expf(-pb));
        dec[tid] = expf(-rate * softplus_f(pa + shift));
      }
    } else {
      for (int i = tid; i < n * DMAX; i += nt) {
        const int tt = i / DMAX, d = i % DMAX;
        const act_t* row = qkv + (size_t)(c0 + tt) * ld + (size_t)g * D;
        qs[i] = d < D ? to_f32(row[d]) : 0.f;
        ks[i] = d < D ? to_f32(row[k_off + d]) : 0.f;
      }
      for (int i = tid; i < n * COLS; i += nt) {
        const int tt = i / COLS, c = i % COLS;
        ov[i] = c < cols ? to_f32(qkv[(size_t)(c0 + tt) * ld + v_off + (size_t)h * E + e0 + c]) : 0.f;
      }
      if (tid < n) {
        const float* row = ba + (size_t)(c0 + tid) * 2 * H;
        beta[tid] = 1.0f / (1.0f + expf(-row[h]));
        dec[tid] = expf(-rate * softplus_f(row[H + h] + shift));
      }
    }
    __syncthreads();
    if (wide && c0 + GRP < t1) fetch(c0 + GRP, min(GRP, t1 - c0 - GRP));
    // unit vectors: 16 lanes a row of q or k, their sum of squares joined inside the lanes' row
    for (int item = tid >> 4; item < 2 * n; item += nt >> 4) {
      float* row = ((item & 1) ? ks : qs) + (item >> 1) * DMAX;
      const int l16 = tid & 15;
      float ss = 0.f;
      for (int d = l16; d < DMAX; d += 16) ss = fmaf(row[d], row[d], ss);
      ss = sum16(ss);
      const float inv = ((item & 1) ? 1.0f : q_scale) / sqrtf(ss + 1e-6f);
      for (int d = l16; d < DMAX; d += 16) row[d] *= inv;
    }
    __syncthreads();
    // the walk: no barrier, three lane permutations a sum.  What the next token needs first (its k, v,
    // beta and decay) is asked for before this token's arithmetic, its q at the token's start.
    float4 kn[CH];
    float vn, bn, gn;
    {
      const float4* k4 = (const float4*)ks + j;
#pragma unroll
      for (int i = 0; i < CH; i++) kn[i] = k4[DS * i];
      vn = ov[col];
      bn = beta[0];
      gn = dec[0];
    }
    for (int tt = 0; tt < n; tt++) {
      const float4* q4 = (const float4*)(qs + tt * DMAX) + j;
      const float gt = gn, bt = bn, vt = vn;
      float4 kk[CH], qq[CH];
#pragma unroll
      for (int i = 0; i < CH; i++) {
        kk[i] = kn[i];
        qq[i] = q4[DS * i];
      }
      if (tt + 1 < n) {
        const float4* k4 = (const float4*)(ks + (tt + 1) * DMAX) + j;
#pragma unroll
        for (int i = 0; i < CH; i++) kn[i] = k4[DS * i];
        vn = ov[(tt + 1) * COLS + col];
        bn = beta[tt + 1];
        gn = dec[tt + 1];
      }
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
      for (int i = 0; i < CH; i++) {
        s[4 * i] *= gt;
        s[4 * i + 1] *= gt;
        s[4 * i + 2] *= gt;
        s[4 * i + 3] *= gt;
        a0 = fmaf(s[4 * i], kk[i].x, a0);
        a1 = fmaf(s[4 * i + 1], kk[i].y, a1);
        a2 = fmaf(s[4 * i + 2], kk[i].z, a2);
        a3 = fmaf(s[4 * i + 3], kk[i].w, a3);
      }
      const float dot = DS == 16 ? sum16((a0 + a1) + (a2 + a3)) : sum8((a0 + a1) + (a2 + a3));
      const float u = bt * (vt - dot);
      a0 = a1 = a2 = a3 = 0.f;
#pragma unroll
      for (int i = 0; i < CH; i++) {
        s[4 * i] = fmaf(kk[i].x, u, s[4 * i]);
        s[4 * i + 1] = fmaf(kk[i].y, u, s[4 * i + 1]);
        s[4 * i + 2] = fmaf(kk[i].z, u, s[4 * i + 2]);
        s[4 * i + 3] = fmaf(kk[i].w, u, s[4 * i + 3]);
        a0 = fmaf(s[4 * i], qq[i].x, a0);
        a1 = fmaf(s[4 * i + 1], qq[i].y, a1);
        a2 = fmaf(s[4 * i + 2], qq[i].z, a2);
        a3 = fmaf(s[4 * i + 3], qq[i].w, a3);
      }
      const float o = DS == 16 ? sum16((a0 + a1) + (a2 + a3)) : sum8((a0 + a1) + (a2 + a3));
      // a column's v of this token was read (by its eight lanes, all in one wave) before the
      // read-out takes its place
      if (j == 0) ov[tt * COLS + col] = o;
    }
    __syncthreads();
    if (raw != nullptr) {                          // the head spans several blocks: its norm comes later
      for (int i = tid; i < n * COLS; i += nt) {
        const int tt = i / COLS, c = i % COLS;
        if (c < cols) raw[((size_t)(c0 + tt) * H + h) * E + e0 + c] = ov[i];
      }
      continue;
    }
    for (int tt = wave; tt < n; tt += nw) {        // unit RMS over the head's read-out, gain, gate
      float ss = 0.f;
      for (int c = lane; c < E; c += 64) ss = fmaf(ov[tt * COLS + c], ov[tt * COLS + c], ss);
      ss = wave_sum(ss);
      const float inv = 1.0f / sqrtf(ss / (float)E + eps);
      const act_t* zr = z + (size_t)(c0 + tt) * ldz + (size_t)h * E;
      act_t* orow = out + ((size_t)(c0 + tt) * H + h) * E;
      for (int c = lane; c < E; c += 64) {
        const float zz = to_f32(zr[c]);
        orow[c] = from_f32<act_t>(ov[tt * COLS + c] * inv * gain[c] * (zz / (1.0f + expf(-zz))));
      }
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < CH; i++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const int d = 4 * (j + DS * i) + c;
        if (d < D) S[(size_t)d * E + e] = s[4 * i + c];
      }
  }
}

// One wave per (token, head): out = raw / sqrt(mean(raw^2) + eps) * gain * silu(z).
__global__ __launch_bounds__(64) void delta_finish_kernel(const float* __restrict__ raw, const act_t* __restrict__ z, int ldz,
                                                          const float* __restrict__ gain, const int* __restrict__ positions,
                                                          act_t* __restrict__ out, int H, int E, float eps) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* rr = raw + ((size_t)t * H + h) * E;
  act_t* orow = out + ((size_t)t * H + h) * E;
  if (positions[t] < 0) {                          // a padding row of a captured step
    for (int c = lane; c < E; c += 64) orow[c] = from_f32<act_t>(0.f);
    return;
  }
  float ss = 0.f;
  for (int c = lane; c < E; c += 64) ss = fmaf(rr[c], rr[c], ss);
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)E + eps);
  const act_t* zr = z + (size_t)t * ldz + (size_t)h * E;
  for (int c = lane; c < E; c += 64) {
    const float zz = to_f32(zr[c]);
    orow[c] = from_f32<act_t>(rr[c] * inv * gain[c] * (zz / (1.0f + expf(-zz))));
  }
}

extern "C" {

// qkv: [T, ld] activations after the convolution and silu: G query heads of D at column 0, G key
// heads at k_off, H value heads of E at v_off.  z: [T, ldz], H heads of E (the output gate before
// its silu).  ba: float [T, 2H], b then a.  A_log, dt_bias: float [H]; gain: float [E].
// state: request r's S [H, D, E] lies at state[slot_of_req[r] * slot_words + offset_words].
// out: [T, H * E].  Requests are rows [q_start[r], q_start[r + 1]).  raw: float scratch [T, H * E],
// used by heads that span several blocks (may be null: a head of up to 128 value channels then stays
// in one block whatever the step); positions: [T].  max_q_len: the longest portion of the step: with
// long portions a block takes 32 value channels, so that a head's walk spreads over more compute units.
int zk_delta_rule(const void* qkv, int ld, int k_off, int v_off, const void* z, int ldz, const float* ba,
                  const float* A_log, const float* dt_bias, const float* gain, float* state, int slot_words,
                  int offset_words, const int* q_start, const int* slot_of_req, const int* positions, void* out,
                  float* raw, int T, int R, int max_q_len, int H, int G, int D, int E, float eps, void* stream) {
  ZK_REQUIRE(T >= 0 && R >= 0 && H > 0 && G > 0 && H % G == 0 && D > 0 && E > 0, "zk_delta_rule: bad sizes");
  ZK_REQUIRE(D <= 256, "zk_delta_rule: up to 256 query/key channels a head");
  ZK_REQUIRE(H <= 65535 && (E + DELTA_COLS_LONG - 1) / DELTA_COLS_LONG <= 65535, "zk_delta_rule: too many heads or value channels");
  ZK_REQUIRE(state != nullptr && slot_words >= offset_words + H * D * E, "zk_delta_rule: the state does not fit its slot");
  const bool scratch = raw != nullptr && positions != nullptr;
  ZK_REQUIRE(E <= DELTA_COLS || scratch, "zk_delta_rule: heads of more than 128 value channels need scratch");
  if (R == 0 || T == 0) return 0;
  const int DMAX = D <= 32 ? 32 : D <= 64 ? 64 : D <= 128 ? 128 : 256;
  // long portions: 16 lanes a column and 16 columns a block, so that a token costs a lane fewer steps
  // and a head spreads over more compute units; the heads' norm then follows in a kernel of its own
  const bool spread = scratch && max_q_len > DELTA_GROUP && E > DELTA_COLS_LONG && DMAX >= 64;
  // (a head of more than 128 rows always has 16 lanes a column: eight would hold more rows each than registers)
  const int DS = (spread || DMAX == 256) ? 16 : 8;
  const int per_block = spread ? DELTA_COLS_LONG : DS == 16 ? DELTA_COLS / 2 : DELTA_COLS;
  ZK_REQUIRE(E <= per_block || scratch, "zk_delta_rule: a head that spans several blocks needs scratch");
  const int blocks_e = (E + per_block - 1) / per_block;
  const int unit = 64 / DS;                                             // columns of a wave
  const int cols = E < per_block ? (E + unit - 1) / unit * unit : per_block;
  const int threads = cols * DS;
  const int GRP = (spread && DMAX <= 128) ? 2 * DELTA_GROUP : DELTA_GROUP;
  const size_t lds = ((size_t)GRP * (2 * DMAX + cols) + 2 * GRP) * sizeof(float);
  // rows in whole groups of eight values at addresses that are whole groups too, and few enough of them a thread
  const int wide = (D % 8 == 0 && E % 8 == 0 && cols % 8 == 0 && ld % 8 == 0 && k_off % 8 == 0 && v_off % 8 == 0 &&
                    (uintptr_t)qkv % 32 == 0 && 2 * GRP * (D / 8) <= (spread ? 4 : 1) * threads && GRP * (cols / 8) <= threads &&
                    GRP <= threads) ? 1 : 0;
  dim3 grid(R, H, blocks_e);
  float* raw_arg = blocks_e > 1 ? raw : nullptr;
#define LAUNCH(C, L, P)                                                                                               \
  delta_rule_kernel<C, L, P><<<grid, threads, lds, (hipStream_t)stream>>>(                                             \
      (const act_t*)qkv, ld, k_off, v_off, (const act_t*)z, ldz, ba, A_log, dt_bias, gain, state, slot_words,         \
      offset_words, q_start, slot_of_req, (act_t*)out, raw_arg, H, G, D, E, eps, cols, GRP, wide)
  if (spread) {                                    // 16 lanes a column, blocks of 256 threads
    if (DMAX == 64) LAUNCH(1, 16, 4);
    else if (DMAX == 128) LAUNCH(2, 16, 4);
    else LAUNCH(4, 16, 4);
  } else if (DS == 8) {
    if (DMAX == 32) LAUNCH(1, 8, 1);
    else if (DMAX == 64) LAUNCH(2, 8, 1);
    else LAUNCH(4, 8, 1);
  } else {
    LAUNCH(4, 16, 1);
  }
#undef LAUNCH
  if (blocks_e > 1) {
    dim3 fg(T, H);
    delta_finish_kernel<<<fg, 64, 0, (hipStream_t)stream>>>(raw, (const act_t*)z, ldz, gain, positions, (act_t*)out, H, E, eps);
  }
  return zk_launch_status("zk_delta_rule");
}

}  // extern "C"

ZK_ENTER(zk_delta_rule)
